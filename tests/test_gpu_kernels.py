"""GPU parity: every kernel-level entry point of the C ABI against the CPU
oracle on the same seeded inputs.

Bars (from the north star): Q8_0 activation quants + scales and per-block int32
dots bit-exact; GEMV float outputs max|err| <= 1e-3 * rms(ref); attention
<= 2e-3 * rms(ref).
"""
import math

import numpy as np
import pytest

import util
from util import Q4_0, Q4_1, Q8_0, Q4_K, Q5_K, Q6_K
from cera_amd import hip_api

pytestmark = pytest.mark.gpu

GEMV_TOL = 1e-3   # x rms(ref)
ATTN_TOL = 2e-3   # x rms(ref)


def _say(msg):
    print(msg, flush=True)


# ---- Q8_0 activation quantizer ------------------------------------------------
@pytest.mark.parametrize("k,scale,seed", [(4096, 1.0, 1), (14336, 1.0, 2), (32, 1.0, 3), (256, 1e-4, 4),
                                          (512, 3e4, 5), (4096 * 8, 0.3, 6)])
def test_quantize_q8_0_bit_exact(hip, orc, k, scale, seed):
    _say(f"quantize k={k} scale={scale} seed={seed}")
    x = util.make_x(k, seed) * np.float32(scale)
    s, q = hip.quantize_q8_0(x)
    s0, q0 = orc.quantize_q8_0(x)
    assert np.array_equal(s.view(np.uint32), s0.view(np.uint32))
    assert np.array_equal(q, q0)


def test_quantize_q8_0_edge_cases_bit_exact(hip, orc):
    _say("quantize edge cases")
    x = util.make_x(32 * 12, 7)
    x[0:32] = 0.0                                   # zero block
    x[32:64] = np.float32(1e-44)                    # subnormal amax -> id = 0
    x[64 + 5] = np.nan                              # NaN lane
    x[96:128] = 0; x[96] = 127.0                    # id == 1 exactly, ties below
    x[97:105] = [0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 3.5, -3.5]
    x[128 + 3] = np.inf                             # inf -> d = inf, id = 0
    x[160:192] = np.float32(1e-38)                  # subnormal-ish d, finite 1/d
    x[192:224] = -np.abs(x[192:224])                # all negative
    x[224:256] = np.float32(3.0e38)                 # huge, d finite, f16 scale = inf
    x[256:288] = np.float32(6e-8) * util.make_x(32, 8)   # scale lands in f16 subnormals
    x[288:320] = np.nan                             # all NaN
    x[320 + 1] = -np.inf
    x[352:384] = np.float32(65504.0 * 127.0)        # f16 scale exactly max finite
    s, q = hip.quantize_q8_0(x)
    s0, q0 = orc.quantize_q8_0(x)
    assert np.array_equal(s.view(np.uint32), s0.view(np.uint32)), (s, s0)
    assert np.array_equal(q, q0)


def test_quantize_rejects_bad_length(hip):
    from cera_amd.hip_api import HipError
    with pytest.raises(HipError):
        hip.quantize_q8_0(np.zeros(33, np.float32))
    with pytest.raises(HipError):
        hip.quantize_q8_0(np.zeros(0, np.float32))


# ---- GEMV ------------------------------------------------------------------------
def _check_gemv(hip, orc, dtype, m, k, seed, debug=True):
    _say(f"gemv {util.NAMES[dtype]} m={m} k={k} seed={seed}")
    w, _ = util.make_weights(dtype, m, k, seed)
    x = util.make_x(k, seed + 1000)
    ref = orc.gemv(dtype, w, x, m, k)
    if debug:
        y, dots, asums = hip.gemv(dtype, w, x, m, k, debug=True)
        _, xq = orc.quantize_q8_0(x)
        dots0, asums0 = orc.block_dots(dtype, w, m, k, xq)
        assert np.array_equal(dots, dots0), "per-block int32 dots differ"
        if dtype in (Q4_1, Q4_K, Q6_K):
            assert np.array_equal(asums, asums0), "activation sums differ"
    y2 = hip.gemv(dtype, w, x, m, k)
    err = np.abs(y2.astype(np.float64) - ref).max()
    assert err <= GEMV_TOL * util.rms(ref), (err, util.rms(ref))
    if debug:
        assert np.array_equal(y.view(np.uint32), y2.view(np.uint32)), "debug and production kernels disagree"
    return err / util.rms(ref)


@pytest.mark.parametrize("dtype", util.INT8_TYPES)
@pytest.mark.parametrize("m,k", [(7, 256), (64, 512), (33, 1024), (130, 4096), (9, 14336), (1, 2048), (5, 11008 // 256 * 256)])
def test_gemv_small_shapes(hip, orc, dtype, m, k):
    _check_gemv(hip, orc, dtype, m, k, seed=dtype * 100 + m)


@pytest.mark.parametrize("dtype", util.INT8_TYPES)
def test_gemv_seeded_shape_sweep(hip, orc, dtype):
    """Seeded random shapes across every K-split width the planner can choose (1..8 wavefronts,
    one and two units per lane), ragged row counts, and -- for the 32-element block types -- K
    that is not a multiple of 256.  Integer dots bit-exact on the smaller ones, floats to the bar."""
    r = util.rng(4000 + dtype)
    step = 256 if dtype in (Q4_K, Q6_K) else 32
    ks = [step * int(v) for v in r.integers(1, 8192 // step + 1, 6)] + [16384 // step * step, 28672 // step * step, 32768]
    for i, k in enumerate(ks):
        m = int(r.integers(1, 300))
        _check_gemv(hip, orc, dtype, m, k, seed=dtype * 1000 + i, debug=(m * k <= 1 << 20))


def test_gemv_config1_q4_0_4096(hip, orc):
    # BASELINE config 1: single Q4_0 GEMV, 4096 x 4096
    rel = _check_gemv(hip, orc, Q4_0, 4096, 4096, seed=11)
    _say(f"  config1 max|err|/rms = {rel:.2e}")


@pytest.mark.parametrize("dtype,m,k", [(Q4_K, 6144, 4096), (Q4_K, 4096, 4096), (Q4_K, 14336, 4096),
                                       (Q6_K, 4096, 14336)])
def test_gemv_config2_llama3_shapes(hip, orc, dtype, m, k):
    rel = _check_gemv(hip, orc, dtype, m, k, seed=21 + m % 97, debug=False)
    _say(f"  {util.NAMES[dtype]} {m}x{k} max|err|/rms = {rel:.2e}")


def test_gemv_config2_head_rows_sampled(hip, orc):
    """Output head 128256 x 4096 Q6_K: full GPU result, oracle on a row sample."""
    m, k = 128256, 4096
    _say("gemv Q6_K head 128256x4096")
    r = util.rng(5)
    base = (r.standard_normal((2048, k)) * 0.02).astype(np.float32)
    wb = util.H.quantize(Q6_K, base, 8).reshape(2048, -1)
    reps = (m + 2047) // 2048
    w = np.ascontiguousarray(np.tile(wb, (reps, 1))[:m])
    # make rows distinct: permute blocks of rows with a roll per repetition
    for i in range(1, reps):
        seg = w[i * 2048:min(m, (i + 1) * 2048)]
        seg[:] = np.roll(wb, i * 7, axis=0)[:seg.shape[0]]
    x = util.make_x(k, 6)
    y = hip.gemv(Q6_K, w.reshape(-1), x, m, k)
    rows = np.unique(np.concatenate([np.arange(0, 64), r.integers(0, m, 512), np.arange(m - 64, m)]))
    ref = orc.gemv(Q6_K, np.ascontiguousarray(w[rows]).reshape(-1), x, rows.size, k)
    err = np.abs(y[rows].astype(np.float64) - ref).max()
    assert err <= GEMV_TOL * util.rms(ref)


def _head_matrix(dtype, m, k, seed):
    """m x k rows built from a 2048-row quantized base, rolled per repetition so rows differ."""
    r = util.rng(seed)
    base = (r.standard_normal((2048, k)) * 0.02).astype(np.float32)
    wb = util.H.quantize(dtype, base, 8).reshape(2048, -1)
    reps = (m + 2047) // 2048
    w = np.empty((m, wb.shape[1]), np.uint8)
    for i in range(reps):
        seg = w[i * 2048:min(m, (i + 1) * 2048)]
        seg[:] = np.roll(wb, i * 7, axis=0)[:seg.shape[0]]
    return w


@pytest.mark.parametrize("dtype", [Q6_K, Q4_K])
def test_head_row_kernel_on_the_decode_copy_at_full_size(hip, orc, no_decode_copies, dtype):
    """The vocabulary head as the decode step launches it -- 128256 x 4096, one wavefront per row
    streaming the decode copy (a Q6_K output.weight, or a tied Q4_K embedding table): every one of
    the 128256 logits carries the bits of the K-split GEMV on the native bytes, the launch from the
    native bytes (copies off) gives the same, and a row sample agrees with the oracle."""
    m, k = 128256, 4096
    _say(f"head row kernel {util.NAMES[dtype]} {m}x{k} on the decode copy")
    w = _head_matrix(dtype, m, k, seed=15)
    x = util.make_x(k, 16)
    y = hip.gemv_store_dev(dtype, w.reshape(-1), x, m, k)
    plain = hip.gemv(dtype, w.reshape(-1), x, m, k)
    assert np.array_equal(y.view(np.uint32), plain.view(np.uint32)), int(np.count_nonzero(y != plain))
    native = no_decode_copies(lambda: hip.gemv_store_dev(dtype, w.reshape(-1), x, m, k))
    assert np.array_equal(y.view(np.uint32), native.view(np.uint32))
    rows = np.unique(np.concatenate([np.arange(0, 64), util.rng(17).integers(0, m, 512), np.arange(m - 64, m)]))
    ref = orc.gemv(dtype, np.ascontiguousarray(w[rows]).reshape(-1), x, rows.size, k)
    assert np.abs(y[rows].astype(np.float64) - ref).max() <= GEMV_TOL * util.rms(ref)


def test_gemv_q5k_f32_activation_path(hip, orc):
    # Q5_K dots against unquantized f32 x on both sides (cpu.rs:1830-1854); row widths that take one,
    # two and four wavefronts per row group, ragged row counts, and a row beyond the K split (20480)
    for m, k in [(9, 512), (64, 4096), (1, 256), (131, 2048), (77, 8192), (100, 14336), (33, 11008), (5, 16384), (6, 20480)]:
        _say(f"gemv Q5_K m={m} k={k}")
        w, _ = util.make_weights(Q5_K, m, k, seed=31 + m)
        x = util.make_x(k, 32)
        y = hip.gemv(Q5_K, w, x, m, k)
        ref = orc.gemv(Q5_K, w, x, m, k)
        assert np.abs(y.astype(np.float64) - ref).max() <= GEMV_TOL * util.rms(ref)
        # and against the exact value: dequantized weights . x in f64
        exact = util.dequant_np(Q5_K, w, m, k).astype(np.float64) @ x.astype(np.float64)
        assert np.abs(y.astype(np.float64) - exact).max() <= GEMV_TOL * util.rms(exact)


def test_gemv_weight_extremes(hip, orc):
    """Q8_0 weights at -128 / 127 against activations at +-127 (simd.rs:6436-6475)."""
    m, k = 8, 256
    _say("gemv Q8_0 extremes")
    blocks = np.zeros((m * k // 32, 34), np.uint8)
    blocks[:, 0:2] = np.array([0.01], np.float16).view(np.uint8)
    q = util.rng(9).integers(-128, 128, size=(m * k // 32, 32)).astype(np.int8)
    q[:, 0:2] = -128
    q[:, 2:4] = 127
    blocks[:, 2:] = q.view(np.uint8)
    x = util.make_x(k, 10)
    x[0::32] = 10.0   # forces +-127 quants at the head of each block
    x[1::32] = 10.0
    x[2::32] = -10.0
    y, dots, _ = hip.gemv(Q8_0, blocks.reshape(-1), x, m, k, debug=True)
    _, xq = orc.quantize_q8_0(x)
    dots0, _ = orc.block_dots(Q8_0, blocks.reshape(-1), m, k, xq)
    assert np.array_equal(dots, dots0)
    ref = orc.gemv(Q8_0, blocks.reshape(-1), x, m, k)
    assert np.abs(y - ref).max() <= GEMV_TOL * util.rms(ref)


def test_gemv_refuses_unsupported(hip):
    from cera_amd.hip_api import HipError
    with pytest.raises(HipError) as e:
        hip.gemv(7, np.zeros(64, np.uint8), np.zeros(32, np.float32), 2, 32)   # unknown ggml type
    assert e.value.status == 3
    with pytest.raises(HipError) as e:
        hip.gemv(Q4_K, np.zeros(144, np.uint8), np.zeros(100, np.float32), 1, 100)  # k not a block multiple
    assert e.value.status == 4
    with pytest.raises(HipError) as e:   # wrong byte count
        hip.gemv(Q4_0, np.zeros(18, np.uint8), np.zeros(64, np.float32), 1, 64)
    assert e.value.status == 4


# ---- glue ops -------------------------------------------------------------------
def test_rmsnorm_bit_exact(hip, orc):
    for n, seed in [(4096, 1), (128, 2), (14336, 3), (256, 4)]:
        _say(f"rmsnorm n={n}")
        x = util.make_x(n, seed) * 3
        w = util.make_x(n, seed + 10)
        y = hip.rmsnorm(x, w, 1e-5)
        ref = orc.rmsnorm(x, w, 1e-5)
        assert np.array_equal(y.view(np.uint32), ref.view(np.uint32))


def test_silu_mul_bit_exact(hip, orc):
    _say("silu_mul")
    g = util.make_x(14336, 5) * 6
    u = util.make_x(14336, 6)
    g[:8] = [0.0, -0.0, 100.0, -100.0, 88.5, -88.5, -104.0, 20.0]
    y = hip.silu_mul(g, u)
    ref = orc.silu_mul(g, u)
    assert np.array_equal(y.view(np.uint32), ref.view(np.uint32))


@pytest.mark.parametrize("norm", [True, False])
def test_rope_bit_exact(hip, orc, norm):
    nh, nkv, hd = 32, 8, 128
    for pos in (0, 1, 17, 511, 4095):
        _say(f"rope norm={norm} pos={pos}")
        q = util.make_x(nh * hd, 40 + pos)
        k = util.make_x(nkv * hd, 41 + pos)
        qa, ka = hip.rope(q, k, pos, nh, nkv, hd, 500000.0, norm)
        qb, kb = orc.rope(q, k, pos, nh, nkv, hd, 500000.0, norm)
        assert np.array_equal(qa.view(np.uint32), qb.view(np.uint32))
        assert np.array_equal(ka.view(np.uint32), kb.view(np.uint32))


def test_argmax_rules(hip, orc):
    _say("argmax")
    r = util.rng(3)
    for n in (1, 7, 1024, 128256):
        x = r.standard_normal(n).astype(np.float32)
        assert hip.argmax(x) == orc.argmax(x)
    x = np.zeros(5000, np.float32); x[[100, 4000, 77]] = 5.0
    assert hip.argmax(x) == 77                         # lowest index on ties
    x = np.full(3000, np.nan, np.float32); x[2500] = -3.0; x[2900] = -3.0
    assert hip.argmax(x) == 2500                       # NaN never wins
    assert hip.argmax(np.full(100, np.nan, np.float32)) == 0
    assert hip.argmax(np.full(100, -np.inf, np.float32)) == 0
    assert hip.argmax(np.zeros(0, np.float32)) == 0


@pytest.mark.parametrize("dtype", util.ALL_TYPES)
def test_dequantize_row_bit_exact(hip, orc, dtype):
    _say(f"dequantize_row {util.NAMES[dtype]}")
    m, k = 6, 1024
    w, _ = util.make_weights(dtype, m, k, seed=50 + dtype, sigma=0.3)
    ref = orc.dequantize(dtype, w, m, k)
    for row in (0, 3, 5):
        out = hip.dequantize_row(dtype, w, m, k, row)
        assert np.array_equal(out.view(np.uint32), ref[row].view(np.uint32))


# ---- decode attention ----------------------------------------------------------------
@pytest.mark.parametrize("L", [1, 2, 63, 64, 65, 512, 1000, 4096, 2560, 5120, 10240, 12289, 16384, 20481])
def test_attn_decode_vs_oracle(hip, orc, L):
    nh, nkv, hd = 32, 8, 128
    _say(f"attn_decode L={L}")
    q = util.make_x(nh * hd, 60)
    k = util.make_x(L * nkv * hd, 61 + L)
    v = util.make_x(L * nkv * hd, 62 + L)
    scale = 1.0 / math.sqrt(hd)
    out = hip.attn_decode(q, k, v, nh, nkv, hd, L, scale)
    ref = orc.decode_attention(q, k, v, nh, nkv, hd, scale, L)
    err = np.abs(out.astype(np.float64) - ref).max()
    assert err <= ATTN_TOL * util.rms(ref), (err, util.rms(ref))


@pytest.mark.parametrize("splits", [1, 3, 16, 1000])
def test_attn_decode_split_invariance(hip, orc, splits):
    nh, nkv, hd, L = 32, 8, 128, 777
    _say(f"attn_decode splits={splits}")
    q = util.make_x(nh * hd, 70)
    k = util.make_x(L * nkv * hd, 71)
    v = util.make_x(L * nkv * hd, 72)
    out = hip.attn_decode(q, k, v, nh, nkv, hd, L, 0.088, n_splits=splits)
    ref = orc.decode_attention(q, k, v, nh, nkv, hd, 0.088, L)
    assert np.abs(out - ref).max() <= ATTN_TOL * util.rms(ref)


@pytest.mark.parametrize("L", [1, 9, 127, 640, 1024, 1025])
def test_attn_decode_auto_matches_explicit_split(hip, L):
    """The automatic split (one 8- or 16-key chunk per wavefront at these lengths) and an explicit
    5-way split give the same result."""
    nh, nkv, hd = 32, 8, 128
    _say(f"attn_decode auto vs 5 splits L={L}")
    q = util.make_x(nh * hd, 75)
    k = util.make_x(L * nkv * hd, 76 + L)
    v = util.make_x(L * nkv * hd, 77 + L)
    auto = hip.attn_decode(q, k, v, nh, nkv, hd, L, 0.09)
    split = hip.attn_decode(q, k, v, nh, nkv, hd, L, 0.09, n_splits=5)
    assert np.isfinite(auto).all()
    assert np.abs(auto - split).max() <= 1e-5 * max(1.0, float(np.abs(split).max()))


def test_attn_decode_peaked_softmax(hip, orc):
    """One dominant key (large logit) and large-magnitude scores: online softmax must not overflow."""
    nh, nkv, hd, L = 8, 2, 128, 300
    _say("attn_decode peaked")
    q = util.make_x(nh * hd, 80) * 4
    k = util.make_x(L * nkv * hd, 81)
    v = util.make_x(L * nkv * hd, 82)
    k.reshape(L, nkv, hd)[200] = q.reshape(nh, hd)[::4] * 2   # aligned with q heads 0 and 4
    out = hip.attn_decode(q, k, v, nh, nkv, hd, L, 1.0)
    ref = orc.decode_attention(q, k, v, nh, nkv, hd, 1.0, L)
    assert np.all(np.isfinite(out))
    assert np.abs(out - ref).max() <= ATTN_TOL * util.rms(ref)


def test_attn_decode_gqa_groupings(hip, orc):
    hd, L = 128, 130
    for nh, nkv in [(8, 8), (8, 4), (16, 2), (4, 1), (28, 4), (12, 2), (6, 2), (5, 1)]:
        _say(f"attn_decode nh={nh} nkv={nkv}")
        q = util.make_x(nh * hd, 90)
        k = util.make_x(L * nkv * hd, 91)
        v = util.make_x(L * nkv * hd, 92)
        out = hip.attn_decode(q, k, v, nh, nkv, hd, L, 0.1)
        ref = orc.decode_attention(q, k, v, nh, nkv, hd, 0.1, L)
        assert np.abs(out - ref).max() <= ATTN_TOL * util.rms(ref)


@pytest.mark.parametrize("nh,nkv,L,n", [(32, 8, 1100, 1), (32, 8, 4200, 1), (32, 8, 9000, 1), (24, 3, 1500, 1), (40, 5, 2300, 1),
                                         (16, 2, 700, 1), (8, 1, 3000, 1), (14, 7, 900, 1), (32, 8, 1200, 5), (24, 3, 2100, 3),
                                         (8, 8, 333, 7), (64, 8, 5000, 2), (16, 2, 17000, 1), (8, 1, 33000, 1),
                                         (28, 4, 3000, 1), (28, 4, 700, 3), (12, 2, 9000, 1), (14, 2, 18000, 1), (6, 2, 1500, 5),
                                         (5, 1, 2500, 1), (28, 4, 200, 40), (12, 2, 1000, 33)])
def test_attn_decode_workgroup_mapping_covers_every_part(hip, orc, nh, nkv, L, n):
    """The partial kernel maps launch indices to (kv head, key range, sub-group of heads, query)
    XCD by XCD and rounds the launch up to whole eights: kv-head counts that do not divide eight,
    part counts that are not multiples of four, both head sub-groups (groups of eight heads keep
    them at every length), group sizes that are not powers of two (Qwen2's 28 / 4 and 12 / 2 heads:
    seven one-head or three two-head wavefronts per kv head; a batch of 16 or more queries takes the
    tiled kernel with one wavefront per head) and small query batches must all reach every
    (head, query), against the oracle query by query."""
    hd = 128
    _say(f"attn workgroup mapping nh={nh} nkv={nkv} L={L} n={n}")
    r = util.rng(31 * L + nh + n)
    q = r.standard_normal((n, nh * hd), dtype=np.float32)
    k = r.standard_normal(L * nkv * hd, dtype=np.float32)
    v = r.standard_normal(L * nkv * hd, dtype=np.float32)
    scale = 1.0 / math.sqrt(hd)
    if n == 1:
        out = hip.attn_decode(q[0], k, v, nh, nkv, hd, L, scale).reshape(1, -1)
    else:
        out = hip.attn_prefill(q, k, v, nh, nkv, hd, L - n, n, scale)
    for i in range(n):
        Li = L - n + i + 1
        ref = orc.decode_attention(q[i], k[:Li * nkv * hd], v[:Li * nkv * hd], nh, nkv, hd, scale, Li)
        err = np.abs(out[i].astype(np.float64) - ref).max()
        assert err <= ATTN_TOL * util.rms(ref), (i, err, util.rms(ref))


@pytest.mark.parametrize("L", [32768, 131072])
def test_attn_decode_config4_long_contexts(hip, orc, L):
    """The long contexts of the flash-decode configuration, against the oracle, plus two
    properties that hold at any size: softmax weights sum to one (a V cache whose rows are all
    the same vector must return that vector) and the result does not depend on how the context
    is split over workgroups."""
    nh, nkv, hd = 32, 8, 128
    _say(f"attn_decode L={L}")
    r = util.rng(1000 + L)
    q = r.standard_normal(nh * hd, dtype=np.float32)
    k = r.standard_normal(L * nkv * hd, dtype=np.float32)
    v = r.standard_normal(L * nkv * hd, dtype=np.float32)
    scale = 1.0 / math.sqrt(hd)
    out = hip.attn_decode(q, k, v, nh, nkv, hd, L, scale)
    ref = orc.decode_attention(q, k, v, nh, nkv, hd, scale, L)
    err = np.abs(out.astype(np.float64) - ref).max()
    _say(f"  max|err|={err:.3e} rms={util.rms(ref):.3e}")
    assert err <= ATTN_TOL * util.rms(ref), (err, util.rms(ref))
    other = hip.attn_decode(q, k, v, nh, nkv, hd, L, scale, n_splits=7)
    assert np.abs(other - out).max() <= 1e-5 * max(1.0, float(np.abs(out).max()))
    row = r.standard_normal(nkv * hd, dtype=np.float32)
    vconst = np.tile(row, L)
    same = hip.attn_decode(q, k, vconst, nh, nkv, hd, L, scale).reshape(nh, hd)
    want = row.reshape(nkv, hd).repeat(nh // nkv, axis=0)
    assert np.abs(same - want).max() <= 2e-6 * float(np.abs(want).max())


# ---- attention over an f16 KV cache ----------------------------------------------------
def _through_half(x):
    return x.astype(np.float16).astype(np.float32)


@pytest.mark.parametrize("L", [1, 9, 65, 512, 1000, 4096, 9000, 20000, 33000])
def test_attn_decode_f16_kv_vs_oracle(hip, orc, L):
    """KvCompression::F16: rows are narrowed to half on append and widened on read
    (cera/src/model/transformer.rs:1170-1196, 1424-1447), so the reference result is the f32
    attention of the half-rounded K and V."""
    nh, nkv, hd = 32, 8, 128
    _say(f"attn_decode f16 kv L={L}")
    q = util.make_x(nh * hd, 160)
    k = util.make_x(L * nkv * hd, 161 + L)
    v = util.make_x(L * nkv * hd, 162 + L)
    scale = 1.0 / math.sqrt(hd)
    out = hip.attn_f16kv(q, k, v, nh, nkv, hd, L - 1, 1, scale).reshape(-1)
    ref = orc.decode_attention(q, _through_half(k), _through_half(v), nh, nkv, hd, scale, L)
    err = np.abs(out.astype(np.float64) - ref).max()
    assert err <= ATTN_TOL * util.rms(ref), (err, util.rms(ref))
    if L >= 65:
        # the rounding is really applied: closer to the half-rounded reference than to the f32 one
        ref32 = orc.decode_attention(q, k, v, nh, nkv, hd, scale, L)
        assert err < np.abs(out.astype(np.float64) - ref32).max()
        other = hip.attn_f16kv(q, k, v, nh, nkv, hd, L - 1, 1, scale, n_splits=3).reshape(-1)
        assert np.abs(other - out).max() <= 1e-5 * max(1.0, float(np.abs(out).max()))


@pytest.mark.parametrize("nh,nkv,start,n", [(32, 8, 0, 96), (8, 2, 300, 40), (16, 2, 1000, 33), (4, 4, 5, 3)])
def test_attn_prefill_f16_kv_vs_oracle(hip, orc, nh, nkv, start, n):
    hd = 128
    _say(f"attn_prefill f16 kv nh={nh} nkv={nkv} start={start} n={n}")
    r = util.rng(11 * n + start)
    L = start + n
    q = r.standard_normal((n, nh * hd), dtype=np.float32)
    k = r.standard_normal(L * nkv * hd, dtype=np.float32)
    v = r.standard_normal(L * nkv * hd, dtype=np.float32)
    scale = 1.0 / np.sqrt(hd)
    out = hip.attn_f16kv(q, k, v, nh, nkv, hd, start, n, scale)
    kh, vh = _through_half(k), _through_half(v)
    for i in sorted(set([0, 1, n // 2, n - 1])):
        Li = start + i + 1
        ref = orc.decode_attention(q[i], kh[:Li * nkv * hd], vh[:Li * nkv * hd], nh, nkv, hd, scale, Li)
        err = np.abs(out[i].astype(np.float64) - ref).max()
        assert err <= ATTN_TOL * util.rms(ref), (i, err, util.rms(ref))


# ---- head_dim 64 (Llama-3.2-1B, Granite-2B, Qwen2 < 7B) ---------------------------------
@pytest.mark.parametrize("kv_f16", [False, True])
@pytest.mark.parametrize("nh,nkv,L", [(32, 8, 1), (32, 8, 777), (8, 8, 130), (16, 2, 5000), (4, 1, 64)])
def test_attn_decode_head_dim_64(hip, orc, kv_f16, nh, nkv, L):
    hd = 64
    _say(f"attn_decode hd=64 nh={nh} nkv={nkv} L={L} f16={kv_f16}")
    q = util.make_x(nh * hd, 260)
    k = util.make_x(L * nkv * hd, 261 + L)
    v = util.make_x(L * nkv * hd, 262 + L)
    scale = 1.0 / math.sqrt(hd)
    if kv_f16:
        out = hip.attn_f16kv(q, k, v, nh, nkv, hd, L - 1, 1, scale).reshape(-1)
        k, v = _through_half(k), _through_half(v)
    else:
        out = hip.attn_decode(q, k, v, nh, nkv, hd, L, scale)
    ref = orc.decode_attention(q, k, v, nh, nkv, hd, scale, L)
    err = np.abs(out.astype(np.float64) - ref).max()
    assert err <= ATTN_TOL * util.rms(ref), (err, util.rms(ref))


# ---- two projections in one launch --------------------------------------------------------
@pytest.mark.parametrize("kv_f16,nh,nkv,hd,L", [(False, 4, 2, 96, 70), (False, 16, 1, 64, 130), (False, 6, 3, 40, 9), (False, 2, 2, 256, 33),
                                               (True, 24, 2, 128, 77), (True, 4, 1, 80, 300)])
def test_attn_decode_other_head_sizes_and_group_sizes(hip, orc, kv_f16, nh, nkv, hd, L):
    """Head sizes other than 64 / 128 and more than 8 query heads per kv head -- which the reference's
    decode_attention takes as it takes any shape (cera/src/model/transformer.rs:1249-1305, kernels
    tested at head_dim 8 ... 256, cera/src/backend/cpu.rs:7075-7088) -- run on the generic kernel:
    same bar against the oracle as the tuned shapes."""
    _say(f"attn decode generic shape heads {nh}/{nkv} hd {hd} L {L} f16={kv_f16}")
    q = util.make_x(nh * hd, 1)
    k, v = util.make_x(L * nkv * hd, 2), util.make_x(L * nkv * hd, 3)
    scale = 1.0 / np.sqrt(hd)
    if kv_f16:
        k, v = k.astype(np.float16).astype(np.float32), v.astype(np.float16).astype(np.float32)
        out = hip.attn_f16kv(q, k, v, nh, nkv, hd, L - 1, 1, scale)[0]
    else:
        out = hip.attn_decode(q, k, v, nh, nkv, hd, L, scale)
    ref = orc.decode_attention(q, k, v, nh, nkv, hd, scale, L)
    assert np.abs(out - ref).max() <= 2e-3 * util.rms(ref)


def test_attn_prefill_other_head_sizes(hip, orc):
    nh, nkv, hd, start, n = 6, 2, 96, 5, 21
    L = start + n
    q = util.make_x(n * nh * hd, 4).reshape(n, nh * hd)
    k, v = util.make_x(L * nkv * hd, 5), util.make_x(L * nkv * hd, 6)
    scale = 1.0 / np.sqrt(hd)
    out = hip.attn_prefill(q, k, v, nh, nkv, hd, start, n, scale)
    for i in (0, 7, n - 1):
        ref = orc.decode_attention(q[i], k, v, nh, nkv, hd, scale, start + i + 1)
        assert np.abs(out[i] - ref).max() <= 2e-3 * util.rms(ref), i


@pytest.mark.parametrize("ma,mb,k", [(5120, 1024, 4096), (4096, 4096, 4096), (1027, 515, 4096), (6, 3, 3072), (70, 30, 1024)])
def test_gemv_pair_is_bitwise_the_two_single_launches(hip, orc, ma, mb, k):
    """attn_q|attn_k (Q4_K) and attn_v (Q6_K) of one layer in a single launch: the same kernel
    body per matrix, so each output equals cera_hip_gemv's bit for bit (and the oracle to the bar)."""
    _say(f"gemv_pair ma={ma} mb={mb} k={k}")
    wa, _ = util.make_weights(Q4_K, ma, k, seed=301)
    wb, _ = util.make_weights(Q6_K, mb, k, seed=302)
    x = util.make_x(k, 303)
    ya, yb = hip.gemv_pair(Q4_K, wa, ma, Q6_K, wb, mb, x, k)
    sa, sb = hip.gemv(Q4_K, wa, x, ma, k), hip.gemv(Q6_K, wb, x, mb, k)
    assert np.array_equal(ya.view(np.uint32), sa.view(np.uint32))
    assert np.array_equal(yb.view(np.uint32), sb.view(np.uint32))
    ref = orc.gemv(Q6_K, wb, x, mb, k)
    assert np.abs(yb - ref).max() <= 1e-3 * util.rms(ref)


def test_gemv_pair_refuses_what_it_has_no_instance_for(hip):
    k = 8192   # a Q4_K row of 8192 takes two wavefronts: no paired instance
    wa, _ = util.make_weights(Q4_K, 8, k, seed=1)
    wb, _ = util.make_weights(Q6_K, 8, k, seed=2)
    with pytest.raises(hip_api.HipError) as e:
        hip.gemv_pair(Q4_K, wa, 8, Q6_K, wb, 8, util.make_x(k, 3), k)
    assert e.value.status == 3
    with pytest.raises(hip_api.HipError) as e:   # types the other way round
        hip.gemv_pair(Q6_K, wb, 8, Q4_K, wa, 8, util.make_x(k, 3), k)
    assert e.value.status == 3


# ---- a few tokens per weight pass ------------------------------------------------------
@pytest.mark.parametrize("dtype", util.INT8_TYPES)
@pytest.mark.parametrize("n", [1, 2, 3, 5, 8, 11, 16])
def test_gemv_multi_token_is_bitwise_per_token_gemv(hip, orc, dtype, n):
    """Short batches go through the multi-token GEMV: every row of the result equals the
    single-vector kernel on that token bit for bit, for every K-split width."""
    # 8200 rows: tall enough for the one-wavefront-per-row multi-token kernel over the decode copy
    for m, k in [(37, 256), (130, 4096), (9, 14336), (260, 1024), (8200, 512)]:
        _say(f"gemv_nb {util.NAMES[dtype]} n={n} m={m} k={k}")
        w, _ = util.make_weights(dtype, m, k, seed=dtype * 31 + n)
        x = util.rng(900 + n).standard_normal((n, k)).astype(np.float32)
        y = hip.gemv_nb(dtype, w, x, m, k)
        for t in range(n):
            one = hip.gemv(dtype, w, x[t], m, k)
            assert np.array_equal(y[t].view(np.uint32), one.view(np.uint32)), (m, k, t)
        ref = orc.gemv(dtype, w, x[n - 1], m, k)
        assert np.abs(y[n - 1] - ref).max() <= GEMV_TOL * util.rms(ref)


def test_gemv_multi_token_refusals(hip):
    with pytest.raises(hip_api.HipError) as e:   # two units per lane: no multi-token instance
        w, _ = util.make_weights(Q4_0, 4, 28672, seed=1)
        hip.gemv_nb(Q4_0, w, np.zeros((2, 28672), np.float32), 4, 28672)
    assert e.value.status == 3


# ---- the decode step's fused kernels, one by one --------------------------------------------------
@pytest.mark.parametrize("n", [4096, 256, 14336, 16384, 32768, 96])
def test_decode_rmsnorm_q8_0_fused_bit_exact(hip, orc, n):
    """The one-launch rmsnorm + Q8_0 quantization of the decode step (the register-resident
    single-row kernel up to 16384 elements, the looping one beyond): normed values, int8 quants and
    scales all carry the bits of cpu::rmsnorm followed by quantize_f32_to_q8_0
    (cera/src/backend/cpu.rs:2479-2496, 942-958)."""
    _say(f"decode rmsnorm+q8_0 n={n}")
    for seed, mag in ((1, 1.0), (2, 40.0), (3, 1e-4)):
        x = util.make_x(n, seed + n) * np.float32(mag)
        w = (1.0 + 0.2 * util.make_x(n, seed + 7)).astype(np.float32)
        y, sc, qq = hip.rmsnorm_q8_0(x, w, 1e-5)
        ref = orc.rmsnorm(x, w, 1e-5)
        rs, rq = orc.quantize_q8_0(ref)
        assert np.array_equal(y.view(np.uint32), ref.view(np.uint32)), (n, seed)
        assert np.array_equal(qq, rq), (n, seed, int(np.count_nonzero(qq != rq)))
        assert np.array_equal(sc.view(np.uint32), rs.view(np.uint32)), (n, seed)


@pytest.mark.parametrize("norm", [True, False])
@pytest.mark.parametrize("kv_f16", [False, True])
@pytest.mark.parametrize("n_heads,n_kv,hd,pos", [(32, 8, 128, 0), (32, 8, 128, 5), (32, 8, 128, 640), (32, 8, 128, 1022),
                                                 (32, 8, 128, 1023), (32, 8, 128, 1500), (8, 2, 64, 37), (8, 8, 64, 1100)])
def test_decode_attention_step_fused_append_and_q8_0(hip, orc, norm, kv_f16, n_heads, n_kv, hd, pos):
    """One decode layer's attention step through the model's own dispatch: the K row it appends
    at `pos` carries the bits of cpu::rope / rope_norm on the new key (cera/src/backend/cpu.rs:
    5008-5180; rounded to half for an f16 cache), the V row those of the new value, whether the
    attention kernel did the rotation and the append itself (below 1024 keys) or a RoPE/append
    launch did; the attention output meets the 2e-3 bar against decode_attention on the rotated
    query and the completed cache; and the Q8_0 output the merge kernel writes for the O
    projection is bit for bit the quantization of that output."""
    _say(f"decode attention step heads {n_heads}/{n_kv} hd {hd} pos {pos} norm={norm} f16={kv_f16}")
    kv_dim = n_kv * hd
    q = util.make_x(n_heads * hd, 11 + pos)
    k_new, v_new = util.make_x(kv_dim, 12 + pos), util.make_x(kv_dim, 13 + pos)
    kc, vc = util.make_x(pos * kv_dim, 14), util.make_x(pos * kv_dim, 15)
    ff = (1.0 + 0.1 * np.arange(hd // 2)).astype(np.float32) if norm and pos % 2 else None
    out, sc, qq, k_row, v_row = hip.attn_decode_step(q, k_new, v_new, kc, vc, n_heads, n_kv, hd, pos, 500000.0, norm=norm,
                                                     freq_factors=ff, kv_f16=kv_f16)
    q_rot, k_rot = orc.rope(q, k_new, pos, n_heads, n_kv, hd, 500000.0, norm=norm, freq_factors=ff)
    half = lambda a: a.astype(np.float16).astype(np.float32)
    k_want, v_want = (half(k_rot), half(v_new)) if kv_f16 else (k_rot, v_new)
    assert np.array_equal(k_row.view(np.uint32), k_want.view(np.uint32)), "appended K row"
    assert np.array_equal(v_row.view(np.uint32), v_want.view(np.uint32)), "appended V row"
    kc_full = np.concatenate([half(kc) if kv_f16 else kc, k_want])
    vc_full = np.concatenate([half(vc) if kv_f16 else vc, v_want])
    ref = orc.decode_attention(q_rot, kc_full, vc_full, n_heads, n_kv, hd, 1.0 / np.sqrt(hd), pos + 1)
    assert np.abs(out - ref).max() <= 2e-3 * util.rms(ref)
    rs, rq = orc.quantize_q8_0(out)
    assert np.array_equal(qq, rq) and np.array_equal(sc.view(np.uint32), rs.view(np.uint32)), "fused Q8_0 of the merge kernel"


# ---- the decode step's fused projection launches ----------------------------------------------------
@pytest.mark.parametrize("ma,mb,k,tb", [(5120, 1024, 4096, Q6_K), (640, 128, 512, Q6_K), (768, None, 256, None),
                                       (96, 64, 2048, Q4_K), (40, 24, 4096, Q6_K)])
def test_qkv_fused_norm_projection(hip, orc, ma, mb, k, tb):
    """attention norm + its Q8_0 quantization + the Q|K (Q4_K) and V projections in one launch:
    every output within the GEMV float bar of the oracle's rmsnorm -> gemv chain
    (cera/src/backend/cpu.rs:2479-2496; cera/src/model/transformer.rs:1340-1373)."""
    _say(f"qkv fused ma={ma} mb={mb} k={k}")
    wa, _ = util.make_weights(Q4_K, ma, k, seed=61)
    wb = util.make_weights(tb, mb, k, seed=62)[0] if mb else None
    x = util.make_x(k, 63) * np.float32(2.5)
    nw = (1.0 + 0.2 * util.make_x(k, 64)).astype(np.float32)
    ya, yb = hip.qkv_fused(Q4_K, wa, ma, tb, wb, mb, k, x, nw, 1e-5)
    n = orc.rmsnorm(x, nw, 1e-5)
    ra = orc.gemv(Q4_K, wa, n, ma, k)
    assert np.abs(ya - ra).max() <= 1e-3 * util.rms(ra)
    if mb:
        rb = orc.gemv(tb, wb, n, mb, k)
        assert np.abs(yb - rb).max() <= 1e-3 * util.rms(rb)


@pytest.mark.parametrize("m,k", [(14336, 4096), (512, 256), (96, 2048), (32, 4096), (18944, 512), (28672, 256)])
def test_ffn_gate_up_fused_against_the_oracle(hip, orc, m, k):
    """FFN norm + Q8_0 + gate | up + SwiGLU + Q8_0 of the result in one launch, against the oracle's
    chain rmsnorm -> gemv x 2 -> silu_mul -> quantize.  The projections agree with the oracle's to
    the float bar only, so a value on a rounding boundary may land one int8 step away and a block
    maximum may round to the neighbouring f16 scale: the dequantized result must meet the oracle's
    SwiGLU output within one quantization step, codes differ by at most one step and rarely."""
    _say(f"ffn gate|up fused m={m} k={k}")
    wg, _ = util.make_weights(Q4_K, m, k, seed=71, sigma=0.05)
    wu, _ = util.make_weights(Q4_K, m, k, seed=72, sigma=0.05)
    x = util.make_x(k, 73) * np.float32(1.7)
    nw = (1.0 + 0.2 * util.make_x(k, 74)).astype(np.float32)
    q, sc = hip.ffn_gate_up_fused(wg, wu, m, k, x, nw, 1e-5)
    n = orc.rmsnorm(x, nw, 1e-5)
    h = orc.silu_mul(orc.gemv(Q4_K, wg, n, m, k), orc.gemv(Q4_K, wu, n, m, k))
    rs, rq = orc.quantize_q8_0(h)
    dq = np.abs(q.astype(np.int32) - rq.astype(np.int32))
    assert dq.max() <= 1 and np.count_nonzero(dq) <= max(2, 0.02 * dq.size), (int(dq.max()), np.count_nonzero(dq))
    ulp = np.abs(sc.astype(np.float16).view(np.int16).astype(np.int32) - rs.astype(np.float16).view(np.int16).astype(np.int32))
    assert np.array_equal(sc, sc.astype(np.float16).astype(np.float32)) and ulp.max() <= 1
    deq = q.astype(np.float32).reshape(-1, 32) * sc[:, None]
    assert (np.abs(deq - h.reshape(-1, 32)) <= 1.01 * rs[:, None] + 1e-9).all()


def test_fused_launches_refuse_what_they_do_not_cover(hip):
    w = np.zeros(8 * 48 * 144, np.uint8)
    with pytest.raises(hip_api.HipError) as e:     # k beyond two passes of a wavefront's 64-weight units
        hip.qkv_fused(Q4_K, w, 8, None, None, None, 12288, np.zeros(12288, np.float32), np.ones(12288, np.float32), 1e-5)
    assert e.value.status == 3
    with pytest.raises(hip_api.HipError) as e:     # m not a whole number of 32-row Q8_0 blocks
        hip.ffn_gate_up_fused(w[:8 * 144], w[:8 * 144], 8, 256, np.zeros(256, np.float32), np.ones(256, np.float32), 1e-5)
    assert e.value.status == 3


def test_ffn_gate_up_fused_is_bitwise_the_separate_launches(hip, orc):
    """The fused launch computes what rmsnorm+Q8_0 -> fused gate|up GEMV -> Q8_0 compute as three
    launches: same activation bytes, same per-row arithmetic, so the same int8 codes and scales."""
    m, k = 2048, 4096
    wg, _ = util.make_weights(Q4_K, m, k, seed=81)
    wu, _ = util.make_weights(Q4_K, m, k, seed=82)
    x = util.make_x(k, 83)
    nw = (1.0 + 0.1 * util.make_x(k, 84)).astype(np.float32)
    q, sc = hip.ffn_gate_up_fused(wg, wu, m, k, x, nw, 1e-5)
    n, _, _ = hip.rmsnorm_q8_0(x, nw, 1e-5)
    h = hip.silu_mul(hip.gemv(Q4_K, wg, n, m, k), hip.gemv(Q4_K, wu, n, m, k))
    rs, rq = hip.quantize_q8_0(h)
    assert np.array_equal(q, rq) and np.array_equal(sc.view(np.uint32), rs.view(np.uint32))


@pytest.mark.parametrize("dtype,m,k", [(Q6_K, 4096, 14336), (Q4_K, 512, 14336), (Q6_K, 77, 8192), (Q4_K, 100, 11008 // 256 * 256),
                                       (Q4_K, 4096, 4096), (Q6_K, 130, 4096), (Q4_K, 33, 256), (Q4_0, 64, 4096)])
def test_projection_with_residual_is_bitwise_the_plain_gemv(hip, dtype, m, k):
    """The decode step's residual projections (O, down) run one wavefront per row where the row
    length allows; whichever kernel a shape takes, y = resid + W.x carries the bits of the plain
    GEMV's W.x added to resid."""
    print(f"projection + residual {util.NAMES[dtype]} {m}x{k}", flush=True)
    w, _ = util.make_weights(dtype, m, k, seed=m + k + 1)
    x = util.make_x(k, 3)
    r = util.make_x(m, 4)
    plain = hip.gemv(dtype, w, x, m, k)
    got = hip.gemv_add_dev(dtype, w, x, r, m, k)
    want = (r + plain).astype(np.float32)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), float(np.abs(got - want).max())


@pytest.fixture
def no_decode_copies(hip):
    """Runs the body with decode copies switched off on the shared context, then on again."""
    def run(fn):
        hip.set_decode_copies(False)
        try:
            return fn()
        finally:
            hip.set_decode_copies(True)
    return run


@pytest.mark.parametrize("dtype,m,k", [(Q6_K, 1024, 14336), (Q4_K, 512, 14336), (Q6_K, 77, 8192), (Q4_K, 100, 6144), (Q4_K, 130, 16384),
                                       (Q4_K, 1030, 4096), (Q6_K, 130, 4096), (Q6_K, 40, 2048), (Q4_K, 33, 1024),
                                       (Q4_K, 70, 3584), (Q6_K, 50, 11008), (Q4_K, 64, 5120), (Q6_K, 40, 256), (Q4_K, 9, 256),
                                       (Q6_K, 35, 3584), (Q4_K, 48, 11008),
                                       (Q4_0, 1030, 4096), (Q8_0, 130, 4096), (Q4_0, 70, 2048), (Q8_0, 33, 1024), (Q4_0, 9, 32),
                                       (Q4_0, 512, 14336), (Q8_0, 200, 14336), (Q4_0, 64, 8192), (Q8_0, 40, 6144), (Q4_0, 50, 11008),
                                       (Q8_0, 24, 4128), (Q4_0, 24, 16384),
                                       (Q4_1, 130, 4096), (Q4_1, 70, 2048), (Q4_1, 64, 14336), (Q4_1, 40, 6144), (Q4_1, 9, 96),
                                       (Q4_K, 130, 8192), (Q6_K, 66, 5120), (Q4_K, 40, 7168), (Q6_K, 70, 18944), (Q4_K, 36, 20480),
                                       (Q6_K, 130, 28672), (Q4_K, 20, 32768), (Q6_K, 12, 24576)])
def test_residual_projection_streams_the_decode_copy_to_the_same_bits(hip, no_decode_copies, dtype, m, k):
    """A matrix's decode copy is a permutation of its bytes, read by the same arithmetic: the
    residual projections give identical bits with the copy (the default) and from the native
    bytes, whatever the row length (planes are padded to whole 128-byte lines)."""
    print(f"decode copy on/off {util.NAMES[dtype]} {m}x{k}", flush=True)
    w, _ = util.make_weights(dtype, m, k, seed=m + k + 7)
    x = util.make_x(k, 5)
    r = util.make_x(m, 6)
    with_copy = hip.gemv_add_dev(dtype, w, x, r, m, k)
    native = no_decode_copies(lambda: hip.gemv_add_dev(dtype, w, x, r, m, k))
    assert np.array_equal(with_copy.view(np.uint32), native.view(np.uint32))
    plain = hip.gemv(dtype, w, x, m, k)
    assert np.array_equal(with_copy.view(np.uint32), (r + plain).astype(np.float32).view(np.uint32))


def test_fused_launches_stream_the_decode_copy_to_the_same_bits(hip, no_decode_copies):
    """The Q|K|V launch (Q4_K and Q6_K matrices in one grid) and the gate|up launch, with and
    without decode copies."""
    k = 4096
    wa, _ = util.make_weights(Q4_K, 1280, k, seed=91)
    wb, _ = util.make_weights(Q6_K, 256, k, seed=92)
    wg, _ = util.make_weights(Q4_K, 1024, k, seed=93)
    wu, _ = util.make_weights(Q4_K, 1024, k, seed=94)
    x = util.make_x(k, 95) * np.float32(1.3)
    nw = (1.0 + 0.1 * util.make_x(k, 96)).astype(np.float32)
    ya, yb = hip.qkv_fused(Q4_K, wa, 1280, Q6_K, wb, 256, k, x, nw, 1e-5)
    q, sc = hip.ffn_gate_up_fused(wg, wu, 1024, k, x, nw, 1e-5)
    ya0, yb0 = no_decode_copies(lambda: hip.qkv_fused(Q4_K, wa, 1280, Q6_K, wb, 256, k, x, nw, 1e-5))
    q0, sc0 = no_decode_copies(lambda: hip.ffn_gate_up_fused(wg, wu, 1024, k, x, nw, 1e-5))
    assert np.array_equal(ya.view(np.uint32), ya0.view(np.uint32)) and np.array_equal(yb.view(np.uint32), yb0.view(np.uint32))
    assert np.array_equal(q, q0) and np.array_equal(sc.view(np.uint32), sc0.view(np.uint32))


@pytest.mark.parametrize("dtype,k", [(Q4_K, 256), (Q4_0, 64), (Q4_1, 96), (Q8_0, 2080)])
@pytest.mark.parametrize("m", [18944, 28672])
def test_gate_up_fused_on_tall_matrices(hip, dtype, k, m):
    """Beyond 64 rows x the CU count the gate|up launch takes 6 (18944 rows) or 8 (28672 rows) rows per
    wavefront instead of a second round of workgroups: bitwise what the separate launches compute,
    for every fused type and for one and two passes per lane."""
    _say(f"gate|up on {m} rows {util.NAMES[dtype]} k={k}")
    wg, _ = util.make_weights(dtype, m, k, seed=121)
    wu, _ = util.make_weights(dtype, m, k, seed=122)
    x = util.make_x(k, 123) * np.float32(1.3)
    nw = (1.0 + 0.1 * util.make_x(k, 124)).astype(np.float32)
    q, sc = hip.ffn_gate_up_fused(wg, wu, m, k, x, nw, 1e-5, dtype)
    n, _, _ = hip.rmsnorm_q8_0(x, nw, 1e-5)
    rs, rq = hip.quantize_q8_0(hip.silu_mul(hip.gemv(dtype, wg, n, m, k), hip.gemv(dtype, wu, n, m, k)))
    assert np.array_equal(q, rq) and np.array_equal(sc.view(np.uint32), rs.view(np.uint32))


@pytest.mark.parametrize("k,tb", [(8192, Q6_K), (5120, Q4_K), (6144, Q6_K)])
def test_fused_launches_for_rows_of_two_passes(hip, orc, no_decode_copies, k, tb):
    """K-quant rows of 4096 < k <= 8192 (the hidden sizes of the 13B - 70B models) take the same fused
    decode launches with two 64-weight units per lane: Q|K|V with the norm inside, gate|up with norm,
    SwiGLU and Q8_0, the O projection with its residual and the head -- bitwise what the separate
    launches compute, with and without decode copies."""
    _say(f"fused launches, two passes per lane, k={k}")
    m = 1024
    wa, _ = util.make_weights(Q4_K, 1280, k, seed=111)
    wb, _ = util.make_weights(tb, 256, k, seed=112)
    wg, _ = util.make_weights(Q4_K, m, k, seed=113)
    wu, _ = util.make_weights(Q4_K, m, k, seed=114)
    x = util.make_x(k, 115) * np.float32(1.3)
    nw = (1.0 + 0.1 * util.make_x(k, 116)).astype(np.float32)
    n, _, _ = hip.rmsnorm_q8_0(x, nw, 1e-5)
    ya, yb = hip.qkv_fused(Q4_K, wa, 1280, tb, wb, 256, k, x, nw, 1e-5)
    assert np.array_equal(ya.view(np.uint32), hip.gemv(Q4_K, wa, n, 1280, k).view(np.uint32))
    assert np.array_equal(yb.view(np.uint32), hip.gemv(tb, wb, n, 256, k).view(np.uint32))
    q, sc = hip.ffn_gate_up_fused(wg, wu, m, k, x, nw, 1e-5)
    rs, rq = hip.quantize_q8_0(hip.silu_mul(hip.gemv(Q4_K, wg, n, m, k), hip.gemv(Q4_K, wu, n, m, k)))
    assert np.array_equal(q, rq) and np.array_equal(sc.view(np.uint32), rs.view(np.uint32))
    ya0, yb0 = no_decode_copies(lambda: hip.qkv_fused(Q4_K, wa, 1280, tb, wb, 256, k, x, nw, 1e-5))
    q0, sc0 = no_decode_copies(lambda: hip.ffn_gate_up_fused(wg, wu, m, k, x, nw, 1e-5))
    assert np.array_equal(ya.view(np.uint32), ya0.view(np.uint32)) and np.array_equal(yb.view(np.uint32), yb0.view(np.uint32))
    assert np.array_equal(q, q0) and np.array_equal(sc.view(np.uint32), sc0.view(np.uint32))
    ref = orc.gemv(Q4_K, wa, orc.rmsnorm(x, nw, 1e-5), 1280, k)
    assert np.abs(ya - ref).max() <= 1e-3 * util.rms(ref)


@pytest.mark.parametrize("dtype,k", [(Q4_0, 4096), (Q8_0, 4096), (Q4_0, 2048), (Q8_0, 1536), (Q4_1, 4096), (Q4_1, 1024)])
def test_fused_launches_for_the_32_block_types(hip, orc, no_decode_copies, dtype, k):
    """Q4_0, Q4_1 and Q8_0 matrices take the same fused decode launches as the K-quants (a lane holds two
    32-weight blocks of a 4096-wide row): Q|K|V with the norm inside and gate|up with norm, SwiGLU and
    Q8_0 -- bitwise what the separate launches compute, with and without decode copies."""
    _say(f"fused launches {util.NAMES[dtype]} k={k}")
    m = 1024
    wa, _ = util.make_weights(dtype, 1280, k, seed=101)
    wg, _ = util.make_weights(dtype, m, k, seed=103)
    wu, _ = util.make_weights(dtype, m, k, seed=104)
    x = util.make_x(k, 105) * np.float32(1.3)
    nw = (1.0 + 0.1 * util.make_x(k, 106)).astype(np.float32)
    ya, _ = hip.qkv_fused(dtype, wa, 1280, None, None, None, k, x, nw, 1e-5)
    q, sc = hip.ffn_gate_up_fused(wg, wu, m, k, x, nw, 1e-5, dtype)
    n, _, _ = hip.rmsnorm_q8_0(x, nw, 1e-5)
    assert np.array_equal(ya.view(np.uint32), hip.gemv(dtype, wa, n, 1280, k).view(np.uint32))
    h = hip.silu_mul(hip.gemv(dtype, wg, n, m, k), hip.gemv(dtype, wu, n, m, k))
    rs, rq = hip.quantize_q8_0(h)
    assert np.array_equal(q, rq) and np.array_equal(sc.view(np.uint32), rs.view(np.uint32))
    ya0, _ = no_decode_copies(lambda: hip.qkv_fused(dtype, wa, 1280, None, None, None, k, x, nw, 1e-5))
    q0, sc0 = no_decode_copies(lambda: hip.ffn_gate_up_fused(wg, wu, m, k, x, nw, 1e-5, dtype))
    assert np.array_equal(ya.view(np.uint32), ya0.view(np.uint32))
    assert np.array_equal(q, q0) and np.array_equal(sc.view(np.uint32), sc0.view(np.uint32))
    ref = orc.gemv(dtype, wa, orc.rmsnorm(x, nw, 1e-5), 1280, k)
    assert np.abs(ya - ref).max() <= 1e-3 * util.rms(ref)
