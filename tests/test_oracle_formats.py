"""Pins the oracle's format layer (cera/src/quant.rs) against independent
implementations and the reference's own known-answer tests."""
import numpy as np
import pytest

import util
from util import Q4_0, Q4_1, Q8_0, Q4_K, Q5_K, Q6_K


def _f32_bits(v: float) -> int:
    return int(np.array([v], np.float32).view(np.uint32)[0])


def test_block_sizes(orc):
    # quant.rs:182,207,223,245,267,293
    want = {Q4_0: (32, 18), Q4_1: (32, 20), Q8_0: (32, 34), Q4_K: (256, 144), Q5_K: (256, 176), Q6_K: (256, 210)}
    for dt, (e, b) in want.items():
        assert orc.lib().orc_block_elems(dt) == e
        assert orc.lib().orc_block_bytes(dt) == b
    assert orc.row_bytes(Q4_K, 4096) == 2304
    assert orc.row_bytes(Q6_K, 4096) == 3360
    assert orc.row_bytes(Q6_K, 14336) == 11760
    assert orc.row_bytes(Q4_0, 4096) * 4096 == 9437184
    assert orc.row_bytes(Q4_K, 100) == 0


def test_f16_widen_exhaustive_vs_numpy(orc):
    # quant.rs:1101-1130: all 65536 patterns against an independent converter.
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32).view(np.uint32)
    L = orc.lib()
    for b in range(65536):
        got = _f32_bits(L.orc_f16_to_f32(b))
        exp, mant = (b >> 10) & 0x1F, b & 0x3FF
        if exp == 0x1F and mant:
            # NaN: payload carried, quiet bit set (quant.rs:62-68)
            assert got == (((b & 0x8000) << 16) | 0x7FC00000 | (mant << 13)), hex(b)
        else:
            assert got == int(want[b]), hex(b)
    assert _f32_bits(L.orc_f16_to_f32(0x7C01)) == 0x7FC02000  # quant.rs:67


def test_bf16_widen(orc):
    L = orc.lib()
    for b in [0, 0x3F80, 0xBF80, 0x7F80, 0xFF80, 0x0001, 0x8001, 0x4049]:
        assert _f32_bits(L.orc_bf16_to_f32(b)) == (b << 16)
    assert _f32_bits(L.orc_bf16_to_f32(0x7F81)) == 0x7FC10000  # sNaN quieted
    assert _f32_bits(L.orc_bf16_to_f32(0xFFC1)) == 0xFFC10000


def test_f32_to_f16_roundtrip_and_boundaries(orc):
    L = orc.lib()
    # every half widened and narrowed back is a fixed point (quant.rs:987-994)
    for b in range(65536):
        v = L.orc_f16_to_f32(b)
        exp, mant = (b >> 10) & 0x1F, b & 0x3FF
        want = b | 0x0200 if (exp == 0x1F and mant) else b
        assert L.orc_f32_to_f16(v) == want, hex(b)
    # boundary floats of quant.rs:1015-1041 against numpy's IEEE converter
    cases = [0.0, -0.0, 1.0, -1.0, np.inf, -np.inf, 65504.0, 65519.0, 65520.0, -65520.0, 1.0e30,
             6.103516e-5, 6.097555e-5, 5.9604645e-8, 2.9802322e-8, 2.9802325e-8, 1.0e-10, -1.0e-10,
             1.0009766, 1.0004883, 1.0014648, 2048.0, 2049.0, 4098.0]
    with np.errstate(over="ignore"):
        for v in cases:
            want = int(np.array([v], np.float32).astype(np.float16).view(np.uint16)[0])
            assert L.orc_f32_to_f16(np.float32(v)) == want, v
    assert L.orc_f32_to_f16(np.float32(65519.0)) == 0x7BFF
    assert L.orc_f32_to_f16(np.float32(65520.0)) == 0x7C00
    assert L.orc_f32_to_f16(np.float32(2.9802322e-8)) == 0x0000
    # NaN narrowing keeps NaN and sets the quiet bit (quant.rs:999-1011)
    for nb in [0x7FC00000, 0xFFC00000, 0x7F800001, 0x7F801000, 0xFF800001]:
        v = np.array([nb], np.uint32).view(np.float32)[0]
        got = L.orc_f32_to_f16(v)
        assert got == (((nb >> 16) & 0x8000) | 0x7E00 | (((nb & 0x7FFFFF) >> 13) & 0x3FF))


def test_f32_to_f16_lcg_sweep_vs_numpy(orc):
    # quant.rs:1043-1056: st = st*1664525 + 1013904223, 200000 draws
    n = 200_000
    st = np.empty(n, np.uint32)
    s = 0x12345678
    for i in range(n):
        s = (s * 1664525 + 1013904223) & 0xFFFFFFFF
        st[i] = s
    vals = st.view(np.float32)
    with np.errstate(over="ignore", invalid="ignore"):
        want = vals.astype(np.float16).view(np.uint16)
    L = orc.lib()
    nan = np.isnan(vals)
    for i in np.nonzero(~nan)[0][::7]:  # every 7th keeps this test fast; all NaN-free classes are hit
        assert L.orc_f32_to_f16(vals[i]) == int(want[i]), hex(int(st[i]))


def test_decode_q4km_scales_known_answer(orc):
    # quant.rs:1848-1878
    sc, mn = orc.decode_q4km_scales(bytes([5, 10, 15, 20, 1, 2, 3, 4, 0, 0, 0, 0]))
    assert list(sc[:4]) == [5, 10, 15, 20] and list(mn[:4]) == [1, 2, 3, 4]
    # high bits: sc[4] = (s[8]&0xF) | (s[0]>>6)<<4 ; mn[4] = (s[8]>>4) | (s[4]>>6)<<4
    sc, mn = orc.decode_q4km_scales(bytes([0xC0 | 1, 0, 0, 0, 0x80 | 2, 0, 0, 0, 0x5A, 0, 0, 0]))
    assert sc[0] == 1 and mn[0] == 2 and sc[4] == (0xA | (3 << 4)) and mn[4] == (0x5 | (2 << 4))


def _h(v):
    return np.array([v], np.float16).view(np.uint8)


def test_dequant_closed_forms(orc):
    # quant.rs:1246-1284
    blk = np.concatenate([_h(1.0), np.full(16, 0x88, np.uint8)])
    assert np.all(orc.dequantize(Q4_0, blk, 1, 32) == 0.0)
    qs = np.array([i | (15 << 4) for i in range(16)], np.uint8)
    out = orc.dequantize(Q4_0, np.concatenate([_h(0.5), qs]), 1, 32)[0]
    assert np.allclose(out[:16], (np.arange(16) - 8) * 0.5) and np.all(out[16:] == 3.5)
    # Q4_1 zero scale keeps the minimum (quant.rs:1214-1223)
    out = orc.dequantize(Q4_1, np.concatenate([_h(0.0), _h(2.5), np.full(16, 0x37, np.uint8)]), 1, 32)
    assert np.all(out == 2.5)
    # Q4_K d=1, dmin=0, sc=1, nibbles 3 -> 3.0 (quant.rs:1532-1567)
    sc = np.array([1, 1, 1, 1, 0, 0, 0, 0, 1, 1, 1, 1], np.uint8)
    blk = np.concatenate([_h(1.0), _h(0.0), sc, np.full(128, 0x33, np.uint8)])
    assert np.all(orc.dequantize(Q4_K, blk, 1, 256) == 3.0)
    # Q6_K ql=0, qh=0xAA, sc=1 -> q = 0 | (2<<4) = 32 -> 0 (quant.rs:1671-1699)
    blk = np.concatenate([np.zeros(128, np.uint8), np.full(64, 0xAA, np.uint8), np.ones(16, np.uint8), _h(1.0)])
    assert np.all(orc.dequantize(Q6_K, blk, 1, 256) == 0.0)
    # Q5_K qs[0]=0x0F, qh[0]=1, sc0=1 -> out[0] = 15 + 16 = 31 (quant.rs:1763-1790)
    qh = np.zeros(32, np.uint8); qh[0] = 1
    qs = np.zeros(128, np.uint8); qs[0] = 0x0F
    blk = np.concatenate([_h(1.0), _h(0.0), sc, qh, qs])
    out = orc.dequantize(Q5_K, blk, 1, 256)[0]
    assert out[0] == 31.0 and np.all(out[1:] == 0.0)


@pytest.mark.parametrize("dtype", util.ALL_TYPES)
def test_dequant_matches_independent_numpy(orc, dtype):
    m, k = 5, 512
    w, _ = util.make_weights(dtype, m, k, seed=100 + dtype, sigma=0.5)
    a = orc.dequantize(dtype, w, m, k)
    b = util.dequant_np(dtype, w, m, k)
    # same formula, possibly different association of d*sc*q: allow 1 ulp-ish
    assert np.allclose(a, b, rtol=3e-7, atol=0), util.NAMES[dtype]


@pytest.mark.parametrize("dtype", util.ALL_TYPES)
def test_random_bytes_dequant_matches_numpy(orc, dtype):
    """Random block bytes (with sane f16 scale fields) exercise every bit position."""
    r = util.rng(7 + dtype)
    e, bsz = util.H.BLOCK[dtype]
    nb = 24
    b = r.integers(0, 256, size=(nb, bsz), dtype=np.uint8)
    scale_fields = {Q4_0: [0], Q4_1: [0, 2], Q8_0: [0], Q4_K: [0, 2], Q5_K: [0, 2], Q6_K: [208]}[dtype]
    for off in scale_fields:
        b[:, off:off + 2] = (r.standard_normal(nb) * 0.1).astype(np.float16).view(np.uint8).reshape(nb, 2)
    a = orc.dequantize(dtype, b.reshape(-1), 1, nb * e)
    ref = util.dequant_np(dtype, b.reshape(-1), 1, nb * e)
    assert np.allclose(a, ref, rtol=3e-7, atol=0)


@pytest.mark.parametrize("dtype", util.ALL_TYPES)
def test_vec_dot_equals_dot_of_dequant(orc, dtype):
    # quant.rs:1286-1306,1633-1669,1701-1733,1792-1823
    k = 512
    w, _ = util.make_weights(dtype, 1, k, seed=3 + dtype, sigma=0.3)
    x = util.make_x(k, 9)
    got = orc.lib().orc_vec_dot_row_f32(dtype, w.ctypes.data, x.ctypes.data, k)
    want = float(util.dequant_np(dtype, w, 1, k)[0].astype(np.float64) @ x.astype(np.float64))
    assert abs(got - want) < 1e-3 * max(1.0, abs(want))
