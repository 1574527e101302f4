"""Pins the oracle's glue ops and decode attention (cera/src/backend/cpu.rs,
cera/src/sampler.rs, cera/src/model/transformer.rs) with closed forms,
invariants and independent numpy/float64 computations."""
import math

import numpy as np
import pytest

import util


def test_expf_close_to_libm_and_saturates(orc):
    # cpu.rs:6547-6567: within ~2 ulp of expf; >88.38 -> inf, < -103.97 -> 0
    xs = np.concatenate([np.linspace(-87, 88, 4001), util.make_x(2000, 1) * 10]).astype(np.float32)
    for x in xs:
        got = orc.expf(float(x))
        want = float(np.exp(np.float64(x)))
        assert abs(got - want) <= 3e-7 * want, x
    assert orc.expf(0.0) == 1.0
    assert math.isinf(orc.expf(89.0)) and orc.expf(200.0) == math.inf
    assert orc.expf(-104.0) == 0.0 and orc.expf(-1000.0) == 0.0
    # gradual range between |n| 126 and 192 stays finite and close
    for x in (-90.0, -100.0, 88.0):  # results below 1.2e-38 are f32 subnormals: one ulp is 1.4e-45
        assert abs(orc.expf(x) - math.exp(x)) <= max(1e-6 * math.exp(x), 1.5e-45)


def test_expf_bit_pattern_of_polynomial(orc):
    """Independent float32 evaluation of the same polynomial in numpy (no FMA)."""
    f = np.float32
    u32 = lambda b: np.array([b], np.uint32).view(np.float32)[0]
    R, LOG2E, HI, LO = u32(0x4B400000), u32(0x3FB8AA3B), u32(0x3F317200), u32(0x35BFBE8E)
    C1, C2, C3, C4, C5 = u32(0x3F7FFFF6), u32(0x3EFFFEDB), u32(0x3E2AAF33), u32(0x3D2B9F17), u32(0x3C072010)
    for x in util.make_x(500, 3) * f(8):
        x = f(x)
        z = f(R + f(x * LOG2E))
        n = f(z - R)
        b = f(f(x - f(n * HI)) - f(n * LO))
        e = (int(np.array([z], np.float32).view(np.uint32)[0]) << 23) & 0xFFFFFFFF
        k = u32((e + 0x3F800000) & 0xFFFFFFFF)
        u = f(b * b)
        j = f(f(C1 * b) + f(f(f(C2 + f(C3 * b)) + f(f(C4 + f(C5 * b)) * u)) * u))
        want = f(k + f(j * k))
        assert np.float32(orc.expf(float(x))).view(np.uint32) == want.view(np.uint32)


def test_rmsnorm_closed_form(orc):
    # cpu.rs:6074-6100: rmsnorm([1,2,3,4], w=1): rms = sqrt(7.5 + eps)
    x = np.array([1, 2, 3, 4], np.float32)
    y = orc.rmsnorm(x, np.ones(4, np.float32), 1e-5)
    assert np.allclose(y, x / math.sqrt(7.5 + 1e-5), rtol=1e-6)
    x = util.make_x(4096, 2)
    w = util.make_x(4096, 3)
    y = orc.rmsnorm(x, w, 1e-5)
    inv = np.float32(1.0 / math.sqrt(float(np.sum(x.astype(np.float64) ** 2)) / 4096 + np.float64(np.float32(1e-5))))
    want = (x * inv) * w
    assert np.array_equal(y.view(np.uint32), want.astype(np.float32).view(np.uint32))


def test_softmax_properties(orc):
    x = util.make_x(1000, 4) * 5
    p = orc.softmax(x)
    assert abs(float(p.sum()) - 1.0) < 1e-5
    ref = np.exp(x.astype(np.float64) - x.max())
    ref /= ref.sum()
    assert np.abs(p - ref).max() < 1e-6
    p = orc.softmax(np.array([1000.0, 1000.0, 999.0], np.float32))  # stability (cpu.rs:6569-6577)
    assert np.all(np.isfinite(p)) and abs(p[0] - p[1]) == 0


def test_silu_mul(orc):
    g = util.make_x(1000, 5) * 4
    u = util.make_x(1000, 6)
    y = orc.silu_mul(g, u)
    ref = g.astype(np.float64) / (1 + np.exp(-g.astype(np.float64))) * u
    assert np.abs(y - ref).max() < 1e-5


def test_argmax_rules(orc):
    # sampler.rs:9-30
    assert orc.argmax(np.array([1, 3, 3, 2], np.float32)) == 1
    assert orc.argmax(np.array([np.nan, 1, np.nan, 5, 5], np.float32)) == 3
    assert orc.argmax(np.array([np.nan, np.nan], np.float32)) == 0
    assert orc.argmax(np.array([], np.float32)) == 0
    assert orc.argmax(np.array([-np.inf, -np.inf], np.float32)) == 0


@pytest.mark.parametrize("norm", [True, False])
def test_rope_properties(orc, norm):
    nh, nkv, hd = 4, 2, 64
    q = util.make_x(nh * hd, 7)
    k = util.make_x(nkv * hd, 8)
    q0, k0 = orc.rope(q, k, 0, nh, nkv, hd, 10000.0, norm)
    assert np.array_equal(q0, q) and np.array_equal(k0, k)  # pos 0 is the identity
    q5, k5 = orc.rope(q, k, 5, nh, nkv, hd, 10000.0, norm)
    # norm preserving per rotated pair
    pairs = (lambda a: a.reshape(-1, hd // 2, 2)) if norm else (lambda a: np.stack([a.reshape(-1, 2, hd // 2)[:, 0], a.reshape(-1, 2, hd // 2)[:, 1]], -1))
    assert np.allclose((pairs(q5) ** 2).sum(-1), (pairs(q) ** 2).sum(-1), rtol=1e-5)
    # closed form for pair i: angle = pos * base^(-2i/hd)
    i = np.arange(hd // 2)
    ang = 5.0 * (10000.0 ** (-2.0 * i / hd))
    x0, x1 = pairs(q)[0, :, 0].astype(np.float64), pairs(q)[0, :, 1].astype(np.float64)
    assert np.allclose(pairs(q5)[0, :, 0], x0 * np.cos(ang) - x1 * np.sin(ang), atol=2e-5)
    assert np.allclose(pairs(q5)[0, :, 1], x0 * np.sin(ang) + x1 * np.cos(ang), atol=2e-5)
    # composition R(3) R(2) = R(5)
    q2, k2 = orc.rope(q, k, 2, nh, nkv, hd, 10000.0, norm)
    q23, _ = orc.rope(q2, k2, 3, nh, nkv, hd, 10000.0, norm)
    assert np.allclose(q23, q5, atol=1e-5)


def test_rope_freq_factors_divide_theta(orc):
    nh, nkv, hd = 1, 1, 8
    q = util.make_x(hd, 9)
    ff = np.array([1, 2, 4, 8], np.float32)
    qa, _ = orc.rope(q, q[:hd], 3, nh, nkv, hd, 100.0, True, ff)
    i = np.arange(hd // 2)
    ang = 3.0 * (100.0 ** (-2.0 * i / hd)) / ff
    x0, x1 = q[0::2].astype(np.float64), q[1::2].astype(np.float64)
    assert np.allclose(qa[0::2], x0 * np.cos(ang) - x1 * np.sin(ang), atol=1e-5)


def attention_f64(q, kc, vc, nh, nkv, hd, scale, L):
    out = np.zeros(nh * hd)
    kc = kc.reshape(L, nkv, hd).astype(np.float64)
    vc = vc.reshape(L, nkv, hd).astype(np.float64)
    for h in range(nh):
        g = h // (nh // nkv)
        s = kc[:, g, :] @ q[h * hd:(h + 1) * hd].astype(np.float64) * scale
        p = np.exp(s - s.max())
        p /= p.sum()
        out[h * hd:(h + 1) * hd] = p @ vc[:, g, :]
    return out


@pytest.mark.parametrize("hd", [8, 24, 64, 72, 128, 256])
def test_decode_attention_variants_vs_f64(orc, hd):
    # cpu.rs:7075-7088 head_dim list (AVX2 kernels vs scalar loops)
    nh, nkv, L = 4, 2, 37
    q = util.make_x(nh * hd, 10)
    kc = util.make_x(L * nkv * hd, 11)
    vc = util.make_x(L * nkv * hd, 12)
    scale = 1.0 / math.sqrt(hd)
    ref = attention_f64(q, kc, vc, nh, nkv, hd, scale, L)
    a = orc.decode_attention(q, kc, vc, nh, nkv, hd, scale, L, variant=0)
    b = orc.decode_attention(q, kc, vc, nh, nkv, hd, scale, L, variant=1)
    assert np.abs(a - ref).max() < 1e-5
    assert np.abs(b - ref).max() < 1e-5
    assert np.abs(a - b).max() < 1e-5


def test_decode_attention_single_position(orc):
    nh, nkv, hd = 8, 2, 128
    q = util.make_x(nh * hd, 13)
    kc = util.make_x(nkv * hd, 14)
    vc = util.make_x(nkv * hd, 15)
    out = orc.decode_attention(q, kc, vc, nh, nkv, hd, 0.1, 1)
    for h in range(nh):
        g = h // 4
        assert np.array_equal(out[h * hd:(h + 1) * hd], vc[g * hd:(g + 1) * hd])
