"""Pins the oracle's Q8_0 activation quantizer and int8 GEMV/GEMM kernels
(cera/src/backend/cpu.rs:942-958, cera/src/backend/simd.rs:4543-6359) against
brute force, the reference's own test fixtures and an independent numpy
restatement."""
import numpy as np
import pytest

import util
from util import Q4_0, Q4_1, Q8_0, Q4_K, Q5_K, Q6_K

MASK64 = (1 << 64) - 1


class Lcg:
    """simd.rs:6421-6426: st = st*6364136223846793005 + 1442695040888963407; st >> 33."""

    def __init__(self, seed):
        self.st = seed & MASK64

    def __call__(self):
        self.st = (self.st * 6364136223846793005 + 1442695040888963407) & MASK64
        return self.st >> 33


def _h(v):
    return np.array([v], np.float32).astype(np.float16).view(np.uint8)


# ---- fixtures restated from simd.rs:6436-6560 ------------------------------
def q8_0_rows_with_extremes(m, k, lcg):
    out = []
    for blk in range(m * (k // 32)):
        out.append(_h(np.float32(0.01) + np.float32(0.003) * np.float32(blk % 5)))
        q = np.empty(32, np.int8)
        for t in range(32):
            if t in (0, 1):
                q[t] = -128
            elif t in (2, 3):
                q[t] = 127
            elif t == 4:
                q[t] = -127
            else:
                q[t] = np.array([lcg() % 256], np.uint8).view(np.int8)[0]
        out.append(q.view(np.uint8))
    return np.concatenate(out)


def q4_0_rows(m, k, lcg):
    out = []
    for blk in range(m * (k // 32)):
        out.append(_h(np.float32(0.01) + np.float32(0.004) * np.float32(blk % 7)))
        out.append(np.array([lcg() % 256 for _ in range(16)], np.uint8))
    return np.concatenate(out)


def q4_1_rows(m, k, lcg):
    out = []
    for blk in range(m * (k // 32)):
        out.append(_h(np.float32(0.01) + np.float32(0.004) * np.float32(blk % 7)))
        out.append(_h(np.float32(-0.05) + np.float32(0.02) * np.float32(blk % 5)))
        out.append(np.array([lcg() % 256 for _ in range(16)], np.uint8))
    return np.concatenate(out)


def k_quant_rows(m, sb, lcg):
    q4 = np.zeros((m * sb, 144), np.uint8)
    for bi in range(m * sb):
        q4[bi, 0:2] = _h(np.float32(0.01) + np.float32(0.005) * np.float32(bi % 7))
        q4[bi, 2:4] = _h(np.float32(0.02) + np.float32(0.003) * np.float32(bi % 5))
        q4[bi, 4:] = [lcg() % 256 for _ in range(140)]
    q6 = np.zeros((m * sb, 210), np.uint8)
    for bi in range(m * sb):
        q6[bi, :208] = [lcg() % 256 for _ in range(208)]
        q6[bi, 208:] = _h(np.float32(0.01) + np.float32(0.004) * np.float32(bi % 6))
    return q4.reshape(-1), q6.reshape(-1)


def activations(n, k, lcg):
    nb = k // 32
    scales = np.zeros((n, nb), np.float32)
    quants = np.zeros((n, k), np.int8)
    for j in range(n):
        for b in range(nb):
            scales[j, b] = np.float32(0.02) + np.float32(0.001) * np.float32((j + b) % 9)
            for t in range(32):
                if t in (0, 1):
                    quants[j, b * 32 + t] = 127
                elif t in (2, 3):
                    quants[j, b * 32 + t] = -127
                else:
                    quants[j, b * 32 + t] = int(lcg() % 255) - 127
    return scales, quants


def ref_gemm_f64(dtype, w, bs, bq, m, n, k):
    """f64 reference sum_b xs*(d*sc*sum q*a - ...) built from independently
    unpacked integer codes (simd.rs:6609-6629, 6847-6877)."""
    q = util.unpack_ints_np(dtype, w, m, k).astype(np.int64)
    e, bsz = util.H.BLOCK[dtype]
    b = w.reshape(-1, bsz)
    out = np.zeros((m, n), np.float64)
    a = bq.astype(np.int64)
    for j in range(n):
        xs = bs[j].astype(np.float64)
        if dtype in (Q4_0, Q8_0):
            d = util._f16(b[:, 0:2]).astype(np.float64).reshape(m, k // 32)
            dots = (q.reshape(m, k // 32, 32) * a[j].reshape(1, k // 32, 32)).sum(-1)
            out[:, j] = (d * xs[None, :] * dots).sum(-1)
        elif dtype == Q4_1:
            d = util._f16(b[:, 0:2]).astype(np.float64).reshape(m, k // 32)
            mm = util._f16(b[:, 2:4]).astype(np.float64).reshape(m, k // 32)
            dots = (q.reshape(m, k // 32, 32) * a[j].reshape(1, k // 32, 32)).sum(-1)
            asum = a[j].reshape(k // 32, 32).sum(-1)
            out[:, j] = (xs[None, :] * (d * dots + mm * asum[None, :])).sum(-1)
        elif dtype == Q4_K:
            d = util._f16(b[:, 0:2]).astype(np.float64).reshape(m, k // 256, 1)
            dmin = util._f16(b[:, 2:4]).astype(np.float64).reshape(m, k // 256, 1)
            sc, mn = util._k_scales(b[:, 4:16])
            sc = sc.astype(np.float64).reshape(m, k // 256, 8)
            mn = mn.astype(np.float64).reshape(m, k // 256, 8)
            dots = (q.reshape(m, k // 256, 8, 32) * a[j].reshape(1, k // 256, 8, 32)).sum(-1)
            asum = a[j].reshape(1, k // 256, 8, 32).sum(-1)
            x8 = xs.reshape(1, k // 256, 8)
            out[:, j] = (x8 * (d * sc * dots - dmin * mn * asum)).sum((-1, -2))
        elif dtype == Q6_K:
            d = util._f16(b[:, 208:210]).astype(np.float64).reshape(m, k // 256, 1)
            sc = b[:, 192:208].view(np.int8).astype(np.float64).reshape(m, k // 256, 16)
            dots = ((q.reshape(m, k // 256, 16, 16) - 32) * a[j].reshape(1, k // 256, 16, 16)).sum(-1)
            x16 = np.repeat(xs, 2).reshape(1, k // 256, 16)
            out[:, j] = (x16 * d * sc * dots).sum((-1, -2))
    return out


# ---- Q8_0 activation quantizer ----------------------------------------------
def quantize_q8_0_np(x):
    """Independent numpy restatement of cpu.rs:942-958 for finite inputs."""
    x = np.asarray(x, np.float32).reshape(-1, 32)
    amax = np.abs(x).max(axis=1).astype(np.float32)
    d = (amax / np.float32(127.0)).astype(np.float32)
    with np.errstate(divide="ignore", over="ignore"):
        r = (np.float32(1.0) / d).astype(np.float32)
    inv = np.where((d != 0) & np.isfinite(r), r, np.float32(0)).astype(np.float32)
    scales = d.astype(np.float16).astype(np.float32)
    q = np.clip(np.rint((x * inv[:, None]).astype(np.float32)), -128, 127).astype(np.int8)
    return scales, q.reshape(-1)


def test_quantize_q8_0_matches_numpy(orc):
    for seed, k, scale in [(1, 4096, 1.0), (2, 14336, 3.0), (3, 256, 1e-3), (4, 64, 1e4)]:
        x = util.make_x(k, seed) * np.float32(scale)
        s, q = orc.quantize_q8_0(x)
        s2, q2 = quantize_q8_0_np(x)
        assert np.array_equal(s.view(np.uint32), s2.view(np.uint32))
        assert np.array_equal(q, q2)
        assert np.abs(q.astype(np.int32)).max() <= 127


def test_quantize_q8_0_edge_cases(orc):
    # simd.rs:7376-7409, 7872-7946 invariants
    x = np.zeros(64, np.float32)
    s, q = orc.quantize_q8_0(x)
    assert np.all(s == 0) and np.all(q == 0)
    # denormal amax: d = amax/127 underflows so 1/d is inf -> id = 0 -> all zero
    x = np.full(32, 1e-44, np.float32)
    s, q = orc.quantize_q8_0(x)
    assert np.all(q == 0) and s[0] == 0.0
    # NaN lane quantizes to 0 and does not poison amax
    x = util.make_x(32, 5)
    x[7] = np.nan
    s, q = orc.quantize_q8_0(x)
    fin = np.delete(x, 7)
    assert q[7] == 0
    assert s[0] == np.float32(np.abs(fin).max() / np.float32(127.0)).astype(np.float16).astype(np.float32)
    # round-half-to-even ties: amax = 127 makes id exactly 1
    x = np.zeros(32, np.float32)
    x[0] = 127.0
    x[1:9] = [0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 3.5, -3.5]
    s, q = orc.quantize_q8_0(x)
    assert list(q[:9]) == [127, 0, 2, 2, 0, -2, -2, 4, -4]
    assert s[0] == 1.0
    # inf input: d = inf, 1/d = 0 (finite) -> id = 0 ... scale is inf, quants 0 (inf*0 = NaN -> 0)
    x = np.zeros(32, np.float32); x[3] = np.inf; x[4] = 1.0
    s, q = orc.quantize_q8_0(x)
    assert np.isinf(s[0]) and np.all(q == 0)


# ---- integer spec -------------------------------------------------------------
@pytest.mark.parametrize("dtype", util.INT8_TYPES)
def test_block_dots_match_numpy_unpack(orc, dtype):
    m, k = 6, 512
    w, _ = util.make_weights(dtype, m, k, seed=40 + dtype)
    _, xq = orc.quantize_q8_0(util.make_x(k, 41))
    dots, asums = orc.block_dots(dtype, w, m, k, xq)
    q = util.unpack_ints_np(dtype, w, m, k).astype(np.int64)
    width = 16 if dtype == Q6_K else 32
    want = (q.reshape(m, k // width, width) * xq.astype(np.int64).reshape(1, k // width, width)).sum(-1)
    assert np.array_equal(dots, want)
    if dtype in (Q4_1, Q4_K, Q6_K):
        assert np.array_equal(asums, xq.astype(np.int64).reshape(k // width, width).sum(-1))


# ---- reference fixtures: integer reference, bound 1e-5 (simd.rs:6584-6700) ----
@pytest.mark.parametrize("variant", [0, 1])
def test_q4_0_q8_0_gemm_matches_integer_reference(orc, variant):
    if variant == 1 and not orc.lib().orc_have_avx2():
        pytest.skip("host has no AVX2+FMA")
    k = 128
    for (m, n) in [(9, 7), (8, 8), (3, 2), (16, 5)]:
        lcg = Lcg(0x1234_5678_9abc_def0 ^ (m * 131 + n))
        w8 = q8_0_rows_with_extremes(m, k, lcg)
        w4 = q4_0_rows(m, k, lcg)
        bs, bq = activations(n, k, lcg)
        for dtype, w in ((Q8_0, w8), (Q4_0, w4)):
            got = orc.gemm_preq(dtype, w, bs, bq, m, n, k, variant)
            want = ref_gemm_f64(dtype, w, bs, bq, m, n, k)
            scale = max(1.0, np.abs(want).max())
            assert np.abs(got - want).max() <= 1e-5 * scale, (util.NAMES[dtype], m, n)


# ---- K-quants + Q4_1: f64 reference, k = 512, bound 1e-4 rel (simd.rs:6847-6919) ----
@pytest.mark.parametrize("variant", [0, 1])
def test_kquant_gemm_matches_f64_reference(orc, variant):
    if variant == 1 and not orc.lib().orc_have_avx2():
        pytest.skip("host has no AVX2+FMA")
    k = 512
    for (m, n) in [(8, 7), (16, 4), (8, 1), (24, 5), (8, 3)]:
        lcg = Lcg(0xfeed_f00d ^ (m * 977 + n))
        q4k, q6k = k_quant_rows(m, k // 256, lcg)
        q41 = q4_1_rows(m, k, lcg)
        bs, bq = activations(n, k, lcg)
        for dtype, w in ((Q4_K, q4k), (Q6_K, q6k), (Q4_1, q41)):
            got = orc.gemm_preq(dtype, w, bs, bq, m, n, k, variant)
            want = ref_gemm_f64(dtype, w, bs, bq, m, n, k)
            scale = max(1.0, np.abs(want).max())
            assert np.abs(got - want).max() <= 1e-4 * scale, (util.NAMES[dtype], m, n)


@pytest.mark.parametrize("dtype", util.INT8_TYPES)
def test_scalar_lane_emulation_equals_avx2_bits(orc, dtype):
    """The two restatements (lane-by-lane scalar, ymm intrinsics) must be the
    same function: same bits at n = 1 (four-accumulator branch) and n > 1."""
    if not orc.lib().orc_have_avx2():
        pytest.skip("host has no AVX2+FMA")
    m, k = 13, 768
    w, _ = util.make_weights(dtype, m, k, seed=60 + dtype)
    for n in (1, 3, 5):
        xs = np.stack([util.make_x(k, 70 + j) for j in range(n)])
        bs = np.empty((n, k // 32), np.float32)
        bq = np.empty((n, k), np.int8)
        for j in range(n):
            bs[j], bq[j] = orc.quantize_q8_0(xs[j])
        a = orc.gemm_preq(dtype, w, bs, bq, m, n, k, 0)
        b = orc.gemm_preq(dtype, w, bs, bq, m, n, k, 1)
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), (util.NAMES[dtype], n)


@pytest.mark.parametrize("dtype", [Q4_0, Q8_0, Q4_1])
def test_decode_equals_prefill_column_bits(orc, dtype):
    """tests/avx2_decode_prefill_identity.rs: for the 32-wide formats a GEMV is
    bit-identical to any column of the GEMM (single accumulator chain)."""
    m, k, n = 7, 512, 4
    w, _ = util.make_weights(dtype, m, k, seed=80 + dtype)
    xs = [((np.array([Lcg(0xa5a50f0f + j)() % 4000 for _ in range(k)], np.float32) / 1000.0) - 2.0) for j in range(n)]
    bs = np.empty((n, k // 32), np.float32)
    bq = np.empty((n, k), np.int8)
    for j in range(n):
        bs[j], bq[j] = orc.quantize_q8_0(xs[j])
    full = orc.gemm_preq(dtype, w, bs, bq, m, n, k)
    for j in range(n):
        y = orc.gemv(dtype, w, xs[j], m, k)
        assert np.array_equal(y.view(np.uint32), full[:, j].copy().view(np.uint32))


@pytest.mark.parametrize("dtype", util.INT8_TYPES)
def test_gemv_vs_dequantized_reference(orc, dtype):
    # cpu.rs:5969-6045: <= 0.02 * max|ref| at m=7, k=256
    m, k = 7, 256
    w, _ = util.make_weights(dtype, m, k, seed=90 + dtype, sigma=0.5)
    x = util.make_x(k, 91)
    y = orc.gemv(dtype, w, x, m, k)
    ref = util.dequant_np(dtype, w, m, k).astype(np.float64) @ x.astype(np.float64)
    assert np.abs(y - ref).max() <= 0.02 * np.abs(ref).max()


@pytest.mark.parametrize("dtype", util.INT8_TYPES)
def test_gemv_matches_f64ref_from_block_dots(orc, dtype):
    m, k = 32, 4096
    w, _ = util.make_weights(dtype, m, k, seed=95 + dtype)
    x = util.make_x(k, 96)
    y = orc.gemv(dtype, w, x, m, k)
    ref = orc.gemv_f64ref(dtype, w, x, m, k)
    assert np.abs(y - ref).max() <= 1e-5 * max(util.rms(ref), 1e-6) * 10


def test_q5k_gemv_is_f32_dot_on_unquantized_x(orc):
    # cpu.rs:1830-1854 + transformer.rs:554-562: no int8 kernel for Q5_K
    m, k = 9, 512
    w, _ = util.make_weights(Q5_K, m, k, seed=11, sigma=0.3)
    x = util.make_x(k, 12)
    y = orc.gemv(Q5_K, w, x, m, k)
    ref = util.dequant_np(Q5_K, w, m, k).astype(np.float64) @ x.astype(np.float64)
    assert np.abs(y - ref).max() <= 1e-4 * max(1.0, np.abs(ref).max())


def test_pool_gemv_equals_serial(orc):
    m, k = 300, 1024
    pool = orc.Pool(4)
    for dtype in util.INT8_TYPES:
        w, _ = util.make_weights(dtype, m, k, seed=20 + dtype)
        x = util.make_x(k, 21)
        a = orc.gemv(dtype, w, x, m, k)
        b = pool.gemv(dtype, w, x, m, k)
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    pool.close()
