"""Pins the oracle's restatement of the x86 prefill route cera runs for Q4_0 / Q4_K weights: the
8-row-interleaved repack and the "8x8" kernels (cera/src/backend/cpu.rs:1145-1421,
cera/src/backend/simd.rs:5215-5518), chosen by transformer::gemm_preq
(cera/src/model/transformer.rs:758-775).  Pins: the reference's own two fixtures and bound
(cpu.rs:5796-5940), the packed layout decoded back by an independent numpy unpacker, a brute
force f64 reference from exact integer dots, and agreement with the standard route."""
import numpy as np
import pytest

import util
from util import Q4_0, Q4_K
from cera_amd import synth

MASK = (1 << 64) - 1


class Lcg:
    """st = st * 6364136223846793005 + 1 (wrapping); value (st >> 33) as u32."""

    def __init__(self, seed):
        self.st = seed

    def __call__(self):
        self.st = (self.st * 6364136223846793005 + 1) & MASK
        return (self.st >> 33) & 0xFFFFFFFF

    def unit(self):   # lcg() as f32 / u32::MAX as f32
        return np.float32(self()) / np.float32(4294967295.0)


def _quantize_cols(orc, lcg, n, k):
    bs = np.empty((n, k // 32), np.float32)
    bq = np.empty((n, k), np.int8)
    for j in range(n):
        col = np.array([lcg.unit() * np.float32(2.0) - np.float32(1.0) for _ in range(k)], np.float32)
        bs[j], bq[j] = orc.quantize_q8_0(col)
    return bs, bq


def _ref_bound(got, want):
    return np.all(np.abs(got - want) <= 1e-4 * np.maximum(np.abs(want), 1.0))


def test_reference_fixture_q4_0_repacked_matches_standard(orc):
    # cpu.rs:5799-5862: (m, n, k) = (16, 13, 128), seed 0xd15ea5ed
    m, n, k = 16, 13, 128
    lcg = Lcg(0xD15EA5ED)
    data = bytearray()
    for _ in range(m * (k // 32)):
        d = np.float16(np.float32(0.01) + np.float32(0.04) * lcg.unit())
        data += d.tobytes()
        data += bytes(lcg() & 0xFF for _ in range(16))
    w = np.frombuffer(bytes(data), np.uint8)
    bs, bq = _quantize_cols(orc, lcg, n, k)
    want = orc.gemm_preq(Q4_0, w, bs, bq, m, n, k)
    got = orc.gemm_8x8(Q4_0, orc.repack_8x8(Q4_0, w, m, k), bs, bq, m, n, k)
    assert _ref_bound(got, want)
    assert np.array_equal(got, orc.gemm_preq_x86(Q4_0, w, bs, bq, m, n, k))   # the dispatcher picks this kernel


def test_reference_fixture_q4_k_repacked_matches_standard(orc):
    # cpu.rs:5871-5940: (16, 13, 256), seed 0x9e3779b9, controlled d / dmin, random scales and nibbles
    m, n, k = 16, 13, 256
    lcg = Lcg(0x9E3779B9)
    data = bytearray()
    for _ in range(m * (k // 256)):
        d = np.float16(np.float32(0.01) + np.float32(0.04) * lcg.unit())
        dmin = np.float16(np.float32(0.02) + np.float32(0.03) * lcg.unit())
        data += d.tobytes() + dmin.tobytes()
        data += bytes(lcg() & 0xFF for _ in range(140))
    w = np.frombuffer(bytes(data), np.uint8)
    bs, bq = _quantize_cols(orc, lcg, n, k)
    want = orc.gemm_preq(Q4_K, w, bs, bq, m, n, k)
    got = orc.gemm_8x8(Q4_K, orc.repack_8x8(Q4_K, w, m, k), bs, bq, m, n, k)
    assert _ref_bound(got, want)
    assert np.array_equal(got, orc.gemm_preq_x86(Q4_K, w, bs, bq, m, n, k))


@pytest.mark.parametrize("dtype,m,k", [(Q4_0, 16, 96), (Q4_0, 8, 32), (Q4_K, 24, 512), (Q4_K, 8, 256)])
def test_packed_layout_decodes_back_to_the_weights(orc, dtype, m, k):
    """packed[(sr*nb + b)*128 + g*16 + i] = row 8sr + i/4 (low nibble) | row 8sr + 4 + i/4 (high) at
    element 4g + i%4 of 32-block b; the baked scales are d (Q4_0) or d*sc, dmin*mn (Q4_K)."""
    w, _ = util.make_weights(dtype, m, k, seed=m * k)
    codes = util.unpack_ints_np(dtype, w, m, k)
    if dtype == Q4_0:
        codes = codes + 8          # the packed layout keeps the raw nibbles
    rp = orc.repack_8x8(dtype, w, m, k)
    nb = k // 32
    packed = rp[0].reshape(m // 8, nb, 8, 16)
    g, i = np.meshgrid(np.arange(8), np.arange(16), indexing="ij")
    e = 4 * g + i % 4
    for sr in range(m // 8):
        for b in range(nb):
            lo = codes[8 * sr + i // 4, 32 * b + e]
            hi = codes[8 * sr + 4 + i // 4, 32 * b + e]
            assert np.array_equal(packed[sr, b] & 0xF, lo) and np.array_equal(packed[sr, b] >> 4, hi)
    blocks = np.ascontiguousarray(w).view(np.uint8).reshape(m, -1)
    if dtype == Q4_0:
        d = blocks.reshape(m, nb, 18)[:, :, :2].copy().view(np.float16).astype(np.float32).reshape(m, nb)
        assert np.array_equal(rp[1].reshape(m // 8, nb, 8), d.reshape(m // 8, 8, nb).transpose(0, 2, 1))
    else:
        sb = blocks.reshape(m, k // 256, 144)
        d = sb[:, :, 0:2].copy().view(np.float16).astype(np.float32).reshape(m, -1)
        dmin = sb[:, :, 2:4].copy().view(np.float16).astype(np.float32).reshape(m, -1)
        sc, mn = util._k_scales(sb[:, :, 4:16].reshape(-1, 12))
        dsc = (d[:, :, None] * sc.reshape(m, -1, 8).astype(np.float32)).reshape(m, nb)
        dmn = (dmin[:, :, None] * mn.reshape(m, -1, 8).astype(np.float32)).reshape(m, nb)
        assert np.array_equal(rp[1].reshape(m // 8, nb, 8), dsc.reshape(m // 8, 8, nb).transpose(0, 2, 1))
        assert np.array_equal(rp[2].reshape(m // 8, nb, 8), dmn.reshape(m // 8, 8, nb).transpose(0, 2, 1))


@pytest.mark.parametrize("dtype", [Q4_0, Q4_K])
@pytest.mark.parametrize("m,n,k", [(8, 7, 512), (16, 4, 512), (8, 1, 512), (24, 5, 512), (8, 3, 1024)])
def test_x86_route_against_f64_reference_and_standard_route(orc, dtype, m, n, k):
    """f64 reference sum_b xs*(d*sc*sum(q a) - dmin*mn*sum(a)) from exact integer dots (the shapes
    and bound of simd.rs:6847-6919), and the reference's own 1e-4 bound against the standard route."""
    w, _ = util.make_weights(dtype, m, k, seed=3 * m + n)
    x = util.rng(m + n + k).standard_normal((n, k)).astype(np.float32)
    bs = np.empty((n, k // 32), np.float32); bq = np.empty((n, k), np.int8)
    for j in range(n):
        bs[j], bq[j] = orc.quantize_q8_0(x[j])
    got = orc.gemm_preq_x86(dtype, w, bs, bq, m, n, k)
    deq = util.dequant_np(dtype, w, m, k).astype(np.float64)
    act = (bq.astype(np.float64).reshape(n, k // 32, 32) * bs.astype(np.float64)[:, :, None]).reshape(n, k)
    ref = deq @ act.T
    assert np.abs(got - ref).max() <= 1e-4 * np.abs(ref).max()
    assert _ref_bound(got, orc.gemm_preq(dtype, w, bs, bq, m, n, k))


def test_x86_route_leaves_other_weights_on_the_standard_route(orc):
    for dtype, m, k in ((util.Q6_K, 16, 256), (util.Q8_0, 16, 64), (Q4_K, 12, 256), (Q4_0, 9, 64)):
        w, _ = util.make_weights(dtype, m, k, seed=1)
        x = util.rng(2).standard_normal((3, k)).astype(np.float32)
        bs = np.empty((3, k // 32), np.float32); bq = np.empty((3, k), np.int8)
        for j in range(3):
            bs[j], bq[j] = orc.quantize_q8_0(x[j])
        assert np.array_equal(orc.gemm_preq_x86(dtype, w, bs, bq, m, 3, k), orc.gemm_preq(dtype, w, bs, bq, m, 3, k))


def test_batched_prefill_through_the_x86_route(orc):
    """The model twin's batched prefill with the repacked kernels tracks the per-token route as
    the standard-layout batched route does (cera/tests/llama_batched_prefill_parity.rs floors)."""
    cfg = dict(synth.TINY)
    weights = synth.make_llama(cfg, seed=5, sigma=0.05, norm_jitter=0.1)
    a, b, c = orc.Llama(cfg, weights), orc.Llama(cfg, weights), orc.Llama(cfg, weights)
    c.set_x86_repack(True)
    toks = [int(t) for t in util.rng(1).integers(0, cfg["vocab"], 12)]
    la = a.forward_prefill_per_token(toks, 0)
    (lb, hb), (lc, hc) = b.forward_prefill_batched(toks, 0, want_hidden=True), c.forward_prefill_batched(toks, 0, want_hidden=True)

    def cos(p, q):
        p, q = p.astype(np.float64), q.astype(np.float64)
        return float(p @ q / np.sqrt((p @ p) * (q @ q)))

    assert cos(la, lc) > 0.9999 and cos(lb, lc) > 0.9999
    # the two routes sum in different orders: bit-identical hidden states would mean the switch did nothing
    assert not np.array_equal(hb, hc) and np.abs(hb - hc).max() <= 0.05 * util.rms(hb)
    for m in (a, b, c):
        m.close()
