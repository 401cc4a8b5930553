"""Pins the C oracle's math helpers against the reference's own known-answer
tests and closed forms (no GPU)."""
import math

import numpy as np
import pytest

from oracle import oracle as orc


# ---- fp16 conversion: independent IEEE implementation = numpy float16 -------
def test_f16_to_f32_all_patterns():
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = np.array([orc.f16_bits_to_f32(int(b)) for b in bits], dtype=np.float32)
    assert np.array_equal(got.view(np.uint32)[~np.isnan(want)], want.view(np.uint32)[~np.isnan(want)])
    assert np.all(np.isnan(got[np.isnan(want)]))


def test_f32_to_f16_rne_subnormals_overflow():
    rng = np.random.default_rng(1)
    vals = np.concatenate([
        rng.normal(0, 1, 20000), rng.normal(0, 1e-5, 20000), rng.normal(0, 3e4, 5000),
        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e9, -1e9, 5.96e-8, 2.98e-8, 2.9802322e-8,
                  2.9802326e-8, 6.1e-5, 6.097e-5, 1.0 + 2 ** -11, 1.0 + 3 * 2 ** -11, 2049.0, 2051.0]),
    ]).astype(np.float32)
    # exact ties between adjacent halves
    halves = np.arange(0, 0x7BFF, 7, dtype=np.uint16).view(np.float16).astype(np.float64)
    nxt = (np.arange(0, 0x7BFF, 7, dtype=np.uint16) + 1).view(np.float16).astype(np.float64)
    ties = ((halves + nxt) / 2).astype(np.float32)
    vals = np.concatenate([vals, ties, -ties])
    want = vals.astype(np.float16).view(np.uint16)
    got = np.array([orc.f32_to_f16_bits(float(v)) for v in vals], dtype=np.uint16)
    assert np.array_equal(got, want)
    assert np.array_equal(orc.round_f16(vals), vals.astype(np.float16).astype(np.float32))


# ---- rmsNorm: Tests/CPUOpsTests/CPUOpsTests.swift:169-208 -------------------
def test_rmsnorm_known_values():
    x = np.array([1, 2, 3, 4, 5, 6, 7, 8], dtype=np.float32).reshape(4, 2)  # channel-first [dim, seq]
    for t in range(2):
        col = x[:, t]
        ss = np.float32(sum(float(v) * float(v) for v in col)) / np.float32(4) + np.float32(1e-5)
        want = col * (1.0 / math.sqrt(ss))
        got = orc.rmsnorm(col, np.ones(4, np.float32), 1e-5)
        assert np.allclose(got, want, atol=1e-5)


def test_rmsnorm_scale_then_weight():
    rng = np.random.default_rng(2)
    x, w = rng.normal(0, 3, 768).astype(np.float32), rng.normal(1, 0.2, 768).astype(np.float32)
    x64 = x.astype(np.float64)
    want = x64 / np.sqrt((x64 * x64).mean() + 1e-5) * w
    assert np.allclose(orc.rmsnorm(x, w, 1e-5), want, rtol=2e-6, atol=1e-7)


# ---- per-head RMSNorm: Tests/CPUOpsTests/RMSNormPerHeadDecodeTests.swift:5-52
def test_per_head_rmsnorm_manual_reference():
    values = np.array([1.0, -2.0, 0.5, 1.5, 2.0, 0.0, -1.0, 3.0], dtype=np.float32)
    weights = np.array([1.0, 0.5, 1.5, 2.0], dtype=np.float32)
    got = orc.per_head_rmsnorm(values, weights, 2, 4, 1e-6)
    for h in range(2):
        v = values[4 * h:4 * h + 4].astype(np.float64)
        want = v / math.sqrt((v * v).sum() / 4 + 1e-6) * weights
        assert np.allclose(got[4 * h:4 * h + 4], want, atol=1e-6)


# ---- RoPE: Tests/CPUOpsTests/RoPEDecodeStepTests.swift:5-45, :48-101, :149-189
def test_rope_half_split_rotation():
    c0, s0, c1, s1 = math.cos(1.0), math.sin(1.0), math.cos(0.01), math.sin(0.01)
    q = orc.rope_half_split([1, 2, 3, 4], 1, 4, 1)
    k = orc.rope_half_split([5, 6, 7, 8], 1, 4, 1)
    assert np.allclose(q, [1 * c0 - 3 * s0, 2 * c1 - 4 * s1, 1 * s0 + 3 * c0, 2 * s1 + 4 * c1], atol=1e-5)
    assert np.allclose(k, [5 * c0 - 7 * s0, 6 * c1 - 8 * s1, 5 * s0 + 7 * c0, 6 * s1 + 8 * c1], atol=1e-5)


def test_rope_position_zero_is_identity_and_theta_matters():
    v = (np.arange(32) % 7 * 0.1 - 0.3).astype(np.float32)
    assert np.array_equal(orc.rope_half_split(v, 4, 8, 0), v)
    a = orc.rope_half_split(v, 4, 8, 5, 10000.0)
    b = orc.rope_half_split(v, 4, 8, 5, 500000.0)
    assert not np.allclose(a, b)
    # first pair has frequency 1 for any theta
    assert np.allclose(a.reshape(4, 8)[:, 0], b.reshape(4, 8)[:, 0])
    # rotation preserves each pair's norm
    av, vv = a.reshape(4, 2, 4), v.reshape(4, 2, 4)
    assert np.allclose((av ** 2).sum(1), (vv ** 2).sum(1), rtol=1e-5)


# ---- attention: RealModelInferenceTests.swift:835-870, HybridDecodeForwardPassTests.swift:97-133
def test_attention_respects_visible_count():
    q = [1, 0]
    k = [1, 100, 0, 0]       # [kvDim=2, stride=2]
    v = [5, 99, 7, 123]
    causal = orc.attention_decode(q, k, v, 1, 1, 2, 1, 2)
    assert causal[0] == 5 and causal[1] == 7
    full = orc.attention_decode(q, k, v, 1, 1, 2, 2, 2)
    assert abs(full[0] - 99) < 0.01 and abs(full[1] - 123) < 0.01


def test_attention_grouped_contiguous_closed_form():
    ctx = orc.attention_decode([1, 2, 3, 4], [1, 2, 0, 1], [10, 20, 30, 40], 2, 1, 2, 2, 2)
    scale = 1 / math.sqrt(2.0)
    want = []
    for logits in ([1 * scale, 4 * scale], [3 * scale, 10 * scale]):
        e = np.exp(np.array(logits) - max(logits))
        p = e / e.sum()
        want += [p @ np.array([10, 20]), p @ np.array([30, 40])]
    assert np.allclose(ctx, want, atol=1e-5)


def test_attention_gqa_groups_map_to_contiguous_kv_heads():
    rng = np.random.default_rng(3)
    heads, kvh, hd, T, S = 8, 2, 16, 11, 16
    q = rng.normal(0, 1, heads * hd).astype(np.float32)
    K = rng.normal(0, 1, (kvh * hd, S)).astype(np.float32)
    V = rng.normal(0, 1, (kvh * hd, S)).astype(np.float32)
    got = orc.attention_decode(q, K, V, heads, kvh, hd, T, S).reshape(heads, hd)
    for h in range(heads):
        kv = h // (heads // kvh)
        Kh, Vh = K[kv * hd:(kv + 1) * hd, :T].astype(np.float64), V[kv * hd:(kv + 1) * hd, :T].astype(np.float64)
        s = q[h * hd:(h + 1) * hd].astype(np.float64) @ Kh / math.sqrt(hd)
        p = np.exp(s - s.max()); p /= p.sum()
        assert np.allclose(got[h], Vh @ p, atol=1e-5)


# ---- SiLU: RealModelInferenceTests.swift:223-229 -----------------------------
def test_silu_tanh_form():
    for s in (-8.0, -1.25, 0.0, 0.75, 6.0):
        assert abs(orc.silu_tanh(s) - 0.5 * s * (1 + math.tanh(0.5 * s))) < 1e-6
        assert abs(orc.silu_tanh(s) - s / (1 + math.exp(-s))) < 1e-6


# ---- matvec ---------------------------------------------------------------
@pytest.mark.parametrize("rows,cols", [(5, 3), (7, 8), (16, 37), (64, 768)])
def test_matvec_against_float64(rows, cols):
    rng = np.random.default_rng(rows * 1000 + cols)
    W, x = rng.normal(0, 1, (rows, cols)).astype(np.float32), rng.normal(0, 1, cols).astype(np.float32)
    want = W.astype(np.float64) @ x.astype(np.float64)
    assert np.allclose(orc.matvec(W, x), want, rtol=1e-5, atol=1e-5)
    # row/column orientation: a one-hot x picks a column
    e = np.zeros(cols, np.float32); e[cols // 2] = 1
    assert np.array_equal(orc.matvec(W, e), W[:, cols // 2])


# ---- argmax: Tests/EspressoTests/PartitionedArgmaxTests.swift:8-115 ----------
def test_partitioned_argmax_row_73_wins_and_prunes():
    vocab, dim = 100, 32
    W = (np.arange(vocab)[:, None] * 0.01 + np.arange(dim)[None, :] * 0.001).astype(np.float32)
    W[73, :] = 10.0
    idx, pruned = orc.partitioned_argmax(W, np.ones(dim, np.float32), block_size=25)
    assert idx == 73 and pruned > 0
    idx1, pruned1 = orc.partitioned_argmax(W, np.ones(dim, np.float32), block_size=4000)
    assert idx1 == 73 and pruned1 == 0


def test_partitioned_argmax_lowest_index_wins_ties_and_matches_naive():
    rng = np.random.default_rng(5)
    W = rng.normal(0, 1, (90, 16)).astype(np.float32)
    W[60] = W[7]                      # exact tie across blocks
    W[8] = W[7]                       # exact tie inside a block
    x = (W[7] * 3).astype(np.float32)
    idx, _ = orc.partitioned_argmax(W, x, block_size=25)
    assert idx == 7
    for seed in range(20):
        r = np.random.default_rng(seed)
        W = r.normal(0, 1, (257, 24)).astype(np.float32)
        x = r.normal(0, 1, 24).astype(np.float32)
        idx, _ = orc.partitioned_argmax(W, x, block_size=40)
        assert idx == int(np.argmax(orc.matvec(W, x)))


# ---- BLOBFILE: WeightBlob.swift:6-18, BlobWeightLoader.swift:62-90 -----------
def test_blobfile_layout_and_errors():
    w = np.array([0.5, -1.25, 3.0, 1e-3], dtype=np.float32)
    blob = orc.blob_build(w)
    assert len(blob) == 128 + 8
    assert blob[0] == 1 and blob[4] == 2 and blob[64:68] == bytes([0xEF, 0xBE, 0xAD, 0xDE]) and blob[68] == 1
    assert int.from_bytes(blob[72:76], "little") == 8 and int.from_bytes(blob[80:84], "little") == 128
    assert np.frombuffer(blob[128:], dtype=np.float16).tolist() == w.astype(np.float16).tolist()
    n, back = orc.blob_parse(blob)
    assert n == 4 and np.array_equal(back, w.astype(np.float16).astype(np.float32))
    assert orc.blob_parse(blob[:100])[0] == -1                       # truncatedHeader
    bad = bytearray(blob); bad[64] = 0
    assert orc.blob_parse(bytes(bad))[0] == -2                       # invalidMagic
    bad = bytearray(blob); bad[80] = 64
    assert orc.blob_parse(bytes(bad))[0] == -3                       # invalidDataOffset
    assert orc.blob_parse(blob[:-2])[0] == -4                        # truncatedPayload
    bad = bytearray(blob); bad[72] = 7
    assert orc.blob_parse(bytes(bad))[0] == -5                       # invalidPayloadSize


# ---- INT4 classifier (Tests/EspressoTests/INT4ClassifierTests.swift) ---------------------------------------
def test_int4_argmax_matches_naive_row_73():            # :8-71
    w = np.zeros((100, 32), np.float32)
    for r in range(100):
        w[r] = np.float32(r) * np.float32(0.01) + np.arange(32, dtype=np.float32) * np.float32(0.001)
    w[73] = 10.0
    x = np.ones(32, np.float32)
    assert int(np.argmax(w @ x)) == 73
    packed, scales, biases = orc.int4_quantize(w)
    assert orc.int4_argmax(packed, scales, biases, x, 32) == 73
    assert scales[73] == 1.0 and biases[73] == 10.0 and not packed[73].any()     # constant row: scale 1, all nibbles 0


def test_int4_matvec_approximation_and_packing():       # :74-131
    w = (np.arange(20 * 16, dtype=np.float32) * np.float32(0.01)).reshape(20, 16)
    x = np.ones(16, np.float32)
    packed, scales, biases = orc.int4_quantize(w)
    got = orc.int4_matvec(packed, scales, biases, x, 16)
    ref = w @ x
    assert np.all(np.abs(got - ref) <= np.abs(ref) * 0.15 + 1.0)
    # closed form of the packing: row r = r*0.16 + 0.01*c, so scale = 0.01 and nibble c = c: bytes (2i << 4) | (2i + 1)
    assert np.allclose(scales, 0.01, rtol=1e-5) and np.allclose(biases, w[:, 0])
    assert packed[0].tolist() == [((2 * i) << 4) | (2 * i + 1) for i in range(8)]
    # dequantised weights are within half a step
    nib = np.stack([packed >> 4, packed & 0xF], axis=2).reshape(20, 16).astype(np.float32)
    assert np.abs(nib * scales[:, None] + biases[:, None] - w).max() <= 0.005 + 1e-5


def test_int4_input_sum_and_odd_dimension():            # :134-173
    assert orc.lib().orc_int4_input_sum is not None
    w = np.full((5, 7), 0.5, np.float32)
    w[3] = 10.0
    packed, scales, biases = orc.int4_quantize(w)
    assert packed.shape == (5, 4) and np.all((packed[:, 3] & 0xF) == 0)          # trailing low nibble is zero
    assert orc.int4_argmax(packed, scales, biases, np.ones(7, np.float32), 7) == 3
    x = np.arange(1, 8, dtype=np.float32)
    mixed = np.random.default_rng(3).normal(0, 1, (9, 7)).astype(np.float32)
    p2, s2, b2 = orc.int4_quantize(mixed)
    nib = np.stack([p2 >> 4, p2 & 0xF], axis=2).reshape(9, 8)[:, :7].astype(np.float64)
    want = (nib * s2[:, None].astype(np.float64) + b2[:, None].astype(np.float64)) @ x.astype(np.float64)
    assert np.allclose(orc.int4_matvec(p2, s2, b2, x, 7), want, rtol=1e-5, atol=1e-5)
