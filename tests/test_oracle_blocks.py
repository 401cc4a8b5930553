"""Pins the oracle's GGUF block codecs.  The reference holds no vector for
them (the arithmetic lives in an absent package), so the pins are: an
independent numpy restatement of the public ggml layouts (bit-exact), an
exhaustive (scale, min, nibble) enumeration, hand-built blocks with known
values, and each format's quantise->dequantise error bound."""
import numpy as np
import pytest

import numpy_ref as ref
from oracle import oracle as orc


def _bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


def test_format_bytes():
    assert orc.format_bytes(orc.FMT_Q8_0, 768 * 768) == 626_688
    assert orc.format_bytes(orc.FMT_Q8_0, 32000 * 768) == 26_112_000
    assert orc.format_bytes(orc.FMT_Q4_K, 4096 * 4096) == 9_437_184
    assert orc.format_bytes(orc.FMT_Q4_0, 4096 * 4096) == 9_437_184
    assert orc.format_bytes(orc.FMT_Q4_K, 14336 * 4096) == 33_030_144


def test_q8_0_hand_built_block():
    blk = np.zeros(34, np.uint8)
    blk[:2] = np.array([0.5], np.float16).view(np.uint8)
    q = np.arange(-16, 16, dtype=np.int8)
    blk[2:] = q.view(np.uint8)
    assert np.array_equal(orc.dequantize(orc.FMT_Q8_0, blk, 32), q.astype(np.float32) * 0.5)


def test_q4_0_hand_built_block_low_nibbles_first_half():
    blk = np.zeros(18, np.uint8)
    blk[:2] = np.array([2.0], np.float16).view(np.uint8)
    lo, hi = np.arange(16, dtype=np.uint8), (15 - np.arange(16)).astype(np.uint8)
    blk[2:] = lo | (hi << 4)
    out = orc.dequantize(orc.FMT_Q4_0, blk, 32)
    assert np.array_equal(out[:16], (lo.astype(np.float32) - 8) * 2)
    assert np.array_equal(out[16:], (hi.astype(np.float32) - 8) * 2)


def test_q4_k_scale_unpack_every_pattern():
    # build a table from known 6-bit values with the packing rule written the other way round
    rng = np.random.default_rng(0)
    for _ in range(200):
        sc, m = rng.integers(0, 64, 8), rng.integers(0, 64, 8)
        t = np.zeros(12, np.uint8)
        for j in range(4):
            t[j] = sc[j] | ((sc[j + 4] >> 4) << 6)
            t[j + 4] = m[j] | ((m[j + 4] >> 4) << 6)
            t[j + 8] = (sc[j + 4] & 0xF) | ((m[j + 4] & 0xF) << 4)
        for j in range(8):
            assert orc.q4_k_scale_min(j, t) == (sc[j], m[j])
        s2, m2 = ref.q4_k_scales_mins(t[None, :])
        assert s2[0].tolist() == sc.tolist() and m2[0].tolist() == m.tolist()


def test_q4_k_hand_built_block():
    blk = np.zeros(144, np.uint8)
    blk[0:2] = np.array([0.25], np.float16).view(np.uint8)
    blk[2:4] = np.array([0.5], np.float16).view(np.uint8)
    sc, m = np.array([1, 2, 3, 4, 33, 34, 35, 63]), np.array([0, 1, 2, 3, 17, 40, 41, 63])
    for j in range(4):
        blk[4 + j] = sc[j] | ((sc[j + 4] >> 4) << 6)
        blk[8 + j] = m[j] | ((m[j + 4] >> 4) << 6)
        blk[12 + j] = (sc[j + 4] & 0xF) | ((m[j + 4] & 0xF) << 4)
    nib = (np.arange(256) * 7 % 16).astype(np.uint8)          # value of weight i
    for c in range(4):
        blk[16 + 32 * c:16 + 32 * c + 32] = nib[64 * c:64 * c + 32] | (nib[64 * c + 32:64 * c + 64] << 4)
    out = orc.dequantize(orc.FMT_Q4_K, blk, 256)
    for j in range(8):
        want = 0.25 * sc[j] * nib[32 * j:32 * j + 32].astype(np.float64) - 0.5 * m[j]   # all exact in fp32
        assert np.array_equal(out[32 * j:32 * j + 32], want.astype(np.float32))


@pytest.mark.parametrize("d,dmin", [(0.0123, 0.0456), (1.0, 1.0), (6.1e-5, 5.96e-8), (65504.0, 0.0), (-0.37, 3.3e-4)])
def test_q4_k_exhaustive_scale_min_nibble(d, dmin):
    """All 64 x 64 x 16 (sc, m, nibble) combinations for a given (d, dmin), bit-exact
    against the numpy restatement (two fp32 roundings, never fused)."""
    blocks = []
    for sc in range(64):
        for m0 in range(0, 64, 8):
            blk = np.zeros(144, np.uint8)
            blk[0:2] = np.array([d], np.float16).view(np.uint8)
            blk[2:4] = np.array([dmin], np.float16).view(np.uint8)
            scs = np.full(8, sc); ms = m0 + np.arange(8)
            for j in range(4):
                blk[4 + j] = scs[j] | ((scs[j + 4] >> 4) << 6)
                blk[8 + j] = ms[j] | ((ms[j + 4] >> 4) << 6)
                blk[12 + j] = (scs[j + 4] & 0xF) | ((ms[j + 4] & 0xF) << 4)
            nib = (np.arange(256) % 16).astype(np.uint8)
            for c in range(4):
                blk[16 + 32 * c:16 + 32 * c + 32] = nib[64 * c:64 * c + 32] | (nib[64 * c + 32:64 * c + 64] << 4)
            blocks.append(blk)
    blocks = np.concatenate(blocks)
    n = blocks.size // 144 * 256
    with np.errstate(over="ignore", invalid="ignore"):
        want = ref.dequant_q4_k(blocks)
    got = orc.dequantize(orc.FMT_Q4_K, blocks, n)
    assert np.array_equal(_bits(got), _bits(want))


@pytest.mark.parametrize("fmt,ref_fn,blk_bytes,blk_len", [
    (orc.FMT_Q8_0, ref.dequant_q8_0, 34, 32), (orc.FMT_Q4_0, ref.dequant_q4_0, 18, 32),
    (orc.FMT_Q4_K, ref.dequant_q4_k, 144, 256)])
def test_dequant_random_bytes_bit_exact_vs_numpy(fmt, ref_fn, blk_bytes, blk_len):
    """Arbitrary block bytes (every scale pattern incl. subnormal/inf/nan halves)."""
    rng = np.random.default_rng(fmt)
    nb = 4096
    blocks = rng.integers(0, 256, nb * blk_bytes, dtype=np.uint8)
    # force edge scales into the first blocks: 0, -0, smallest subnormal, max half, inf
    edge = np.array([0x0000, 0x8000, 0x0001, 0x7BFF, 0x7C00, 0x03FF, 0x0400, 0xFBFF], np.uint16)
    for i, e in enumerate(edge):
        blocks[i * blk_bytes:i * blk_bytes + 2] = np.array([e], np.uint16).view(np.uint8)
    with np.errstate(over="ignore", invalid="ignore"):
        want = ref_fn(blocks)
    got = orc.dequantize(fmt, blocks, nb * blk_len)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(_bits(got)[~nan], _bits(want)[~nan])


def test_quantize_error_bounds_and_layout():
    rng = np.random.default_rng(7)
    x = rng.normal(0, 0.02, 64 * 256).astype(np.float32)
    # Q8_0: |x - dq| <= d/2 + 127*|d - fp16(d)|
    b = orc.quantize(orc.FMT_Q8_0, x)
    dq = orc.dequantize(orc.FMT_Q8_0, b, x.size)
    amax = np.abs(x.reshape(-1, 32)).max(1)
    d = amax / 127
    bound = (d / 2 + 127 * d * 2.0 ** -11 + 1e-12)[:, None]
    assert np.all(np.abs(dq - x).reshape(-1, 32) <= bound)
    d16 = b.reshape(-1, 34)[:, :2].copy().view(np.float16).ravel()
    assert np.array_equal(d16, d.astype(np.float32).astype(np.float16))
    # Q4_0: the largest-magnitude element maps to nibble 0 (-8*d); everything within d (clipped top)
    b = orc.quantize(orc.FMT_Q4_0, x)
    dq = orc.dequantize(orc.FMT_Q4_0, b, x.size)
    assert np.all(np.abs(dq - x).reshape(-1, 32) <= (amax / 8 * 1.01)[:, None])
    # Q4_K: within one step of the widest sub-block
    b = orc.quantize(orc.FMT_Q4_K, x)
    dq = orc.dequantize(orc.FMT_Q4_K, b, x.size)
    span = x.reshape(-1, 256).max(1) - np.minimum(x.reshape(-1, 256).min(1), 0)
    assert np.all(np.abs(dq - x).reshape(-1, 256) <= (span / 15 * 1.1)[:, None])
    rel = np.linalg.norm(dq - x) / np.linalg.norm(x)
    assert rel < 0.12
    # zero input
    z = np.zeros(256, np.float32)
    for fmt in (orc.FMT_Q8_0, orc.FMT_Q4_0, orc.FMT_Q4_K):
        assert np.array_equal(orc.dequantize(fmt, orc.quantize(fmt, z), 256), z)


def test_f16_and_f32_formats_round_trip():
    x = np.random.default_rng(8).normal(0, 0.02, 512).astype(np.float32)
    assert np.array_equal(orc.dequantize(orc.FMT_F32, orc.quantize(orc.FMT_F32, x), 512), x)
    assert np.array_equal(orc.dequantize(orc.FMT_F16, orc.quantize(orc.FMT_F16, x), 512),
                          x.astype(np.float16).astype(np.float32))
