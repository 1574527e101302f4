"""GPU parity for the prefill path: int8-MFMA GEMM vs the oracle's gemm_preq on
the same Q8_0-quantized activations, and batched prefill of a small llama vs
the oracle's forward_prefill_batched."""
import numpy as np
import pytest

import util
from util import Q4_0, Q4_1, Q8_0, Q4_K, Q5_K, Q6_K
from cera_amd import hip_api, synth

pytestmark = pytest.mark.gpu
GEMM_TOL = 1e-3  # x rms(ref), the north star's bar for GEMM


def _say(msg):
    print(msg, flush=True)


def _oracle_gemm(orc, dtype, w, x, m, n, k):
    bs = np.empty((n, k // 32), np.float32)
    bq = np.empty((n, k), np.int8)
    for j in range(n):
        bs[j], bq[j] = orc.quantize_q8_0(x[j])
    return orc.gemm_preq(dtype, w, bs, bq, m, n, k)


@pytest.mark.parametrize("dtype", util.INT8_TYPES)
@pytest.mark.parametrize("m,n,k", [(128, 64, 256), (7, 3, 512), (200, 65, 1024), (130, 1, 256), (64, 130, 4096)])
def test_gemm_small_shapes(hip, orc, dtype, m, n, k):
    _say(f"gemm {util.NAMES[dtype]} m={m} n={n} k={k}")
    w, _ = util.make_weights(dtype, m, k, seed=dtype * 10 + m)
    x = util.rng(dtype + n).standard_normal((n, k)).astype(np.float32)
    out = hip.gemm(dtype, w, x, m, n, k)
    ref = _oracle_gemm(orc, dtype, w, x, m, n, k)
    err = np.abs(out.astype(np.float64) - ref).max()
    assert err <= GEMM_TOL * util.rms(ref), (err, util.rms(ref))


@pytest.mark.parametrize("dtype", util.INT8_TYPES)
def test_gemm_seeded_shape_sweep(hip, orc, dtype):
    """Seeded random (rows, tokens, k): ragged tiles on both sides, and few output tiles with a long
    K so the split-K route and its fixed-order reduction are exercised."""
    r = util.rng(5000 + dtype)
    shapes = [(int(r.integers(1, 400)), int(r.integers(1, 200)), 256 * int(r.integers(1, 17))) for _ in range(5)]
    shapes += [(64, 48, 8192), (130, 17, 14336), (256, 64, 4096)]
    for m, n, k in shapes:
        _say(f"gemm sweep {util.NAMES[dtype]} m={m} n={n} k={k}")
        w, _ = util.make_weights(dtype, m, k, seed=dtype * 7 + m)
        x = util.rng(m + n).standard_normal((n, k)).astype(np.float32)
        out = hip.gemm(dtype, w, x, m, n, k)
        ref = _oracle_gemm(orc, dtype, w, x, m, n, k)
        err = np.abs(out.astype(np.float64) - ref).max()
        assert err <= GEMM_TOL * util.rms(ref), (m, n, k, err, util.rms(ref))


@pytest.mark.parametrize("dtype,m,k", [(Q4_K, 4096, 4096), (Q6_K, 4096, 14336)])
@pytest.mark.parametrize("n", [128, 512, 2048])
def test_gemm_config3_shapes_row_sample(hip, orc, dtype, m, k, n):
    """BASELINE config 3 shapes; the oracle checks a sample of output rows."""
    _say(f"gemm {util.NAMES[dtype]} m={m} n={n} k={k}")
    w, _ = util.make_weights(dtype, m, k, seed=3)
    x = util.rng(n).standard_normal((n, k)).astype(np.float32)
    out = hip.gemm(dtype, w, x, m, n, k)
    rows = np.unique(np.concatenate([np.arange(8), util.rng(1).integers(0, m, 40), np.arange(m - 8, m)]))
    rb = util.H.row_bytes(dtype, k)
    wr = np.ascontiguousarray(w.reshape(m, rb)[rows]).reshape(-1)
    ref = _oracle_gemm(orc, dtype, wr, x, rows.size, n, k)
    err = np.abs(out[rows].astype(np.float64) - ref).max()
    assert err <= GEMM_TOL * util.rms(ref), (err, util.rms(ref))


def test_gemm_equals_gemv_per_column(hip, orc):
    """decode == prefill at the GEMM level: every column of the GEMM agrees with the
    GEMV of that token (tests/avx2_decode_prefill_identity.rs, to the float bar)."""
    m, n, k = 96, 5, 1024
    for dtype in (Q4_K, Q6_K, Q4_0):
        w, _ = util.make_weights(dtype, m, k, seed=9)
        x = util.rng(7).standard_normal((n, k)).astype(np.float32)
        out = hip.gemm(dtype, w, x, m, n, k)
        for j in range(n):
            y = hip.gemv(dtype, w, x[j], m, k)
            assert np.abs(out[:, j] - y).max() <= 2e-5 * max(util.rms(y), 1e-6) * 10


@pytest.mark.parametrize("dtype", [Q4_K, Q6_K, Q4_0])
@pytest.mark.parametrize("ma,mb,n,k", [(256, 128, 40, 512), (4096, 1024, 512, 4096), (300, 77, 33, 2048),
                                       (1024, 1024, 1100, 256)])
def test_gemm_pair_matches_single_launches(hip, orc, dtype, ma, mb, n, k):
    """Q|K and gate|up share a launch in the prefill pass: each output equals the matrix's own GEMM
    (bit for bit where neither launch splits K; to the order of the partial sums where they do,
    as at 4096 x 4096 | 1024 x 4096 with 512 tokens), and a row sample agrees with the oracle."""
    _say(f"gemm pair {util.NAMES[dtype]} ma={ma} mb={mb} n={n} k={k}")
    wa, _ = util.make_weights(dtype, ma, k, seed=31)
    wb, _ = util.make_weights(dtype, mb, k, seed=32)
    x = util.rng(n + k).standard_normal((n, k)).astype(np.float32)
    oa, ob = hip.gemm_pair(dtype, wa, ma, dtype, wb, mb, x, n, k)
    sa, sb = hip.gemm(dtype, wa, x, ma, n, k).T, hip.gemm(dtype, wb, x, mb, n, k).T
    for got, single in ((oa, sa), (ob, sb)):
        assert np.abs(got - single).max() <= 2e-5 * util.rms(single)
    rows = np.unique(np.concatenate([np.arange(4), np.arange(mb - 4, mb)]))
    rb = util.H.row_bytes(dtype, k)
    wr = np.ascontiguousarray(wb.reshape(mb, rb)[rows]).reshape(-1)
    ref = _oracle_gemm(orc, dtype, wr, x, rows.size, n, k)
    assert np.abs(ob[:, rows].T.astype(np.float64) - ref).max() <= GEMM_TOL * util.rms(ref)


@pytest.mark.parametrize("dtype", [Q4_K, Q4_0, Q4_1, Q8_0])
@pytest.mark.parametrize("m,k,n,want_fused", [(2048, 512, 1040, True), (1056, 256, 2000, True), (512, 256, 70, False)])
def test_gemm_swiglu_epilogue_matches_separate_kernels(hip, orc, dtype, m, k, n, want_fused):
    """gate | up | SwiGLU | Q8_0 in one launch: the quants and scales must be, byte for byte, the
    oracle's quantization of the oracle's SwiGLU of the two GEMM outputs the pair launch gives
    (silu_mul_inplace cpu.rs:2570-2575, quantize_columns transformer.rs:865-946).  Row counts
    that are not a multiple of the 64-row tile, ragged token tiles, and a batch too small to
    fill the chip (which takes the separate kernels) are covered."""
    _say(f"gemm_swiglu {util.NAMES[dtype]} m={m} k={k} n={n}")
    wg, _ = util.make_weights(dtype, m, k, seed=41)
    wu, _ = util.make_weights(dtype, m, k, seed=42)
    x = util.rng(m + 3 * n).standard_normal((n, k)).astype(np.float32)
    q, sc, fused = hip.gemm_swiglu(dtype, wg, wu, m, x, n, k)
    assert fused == want_fused
    g, u = hip.gemm_pair(dtype, wg, m, dtype, wu, m, x, n, k)
    h = orc.silu_mul(g.reshape(-1), u.reshape(-1))
    ref_s, ref_q = orc.quantize_q8_0(h)
    assert np.array_equal(q.reshape(-1), ref_q)
    assert np.array_equal(sc.reshape(-1).view(np.uint32), ref_s.view(np.uint32))


@pytest.mark.parametrize("dtype,m,k,n,want_fused", [(Q4_K, 2048, 512, 1040, True), (Q4_K, 1056, 256, 2000, True),
                                                      (Q4_K, 512, 256, 80, False), (Q4_0, 2048, 512, 1040, True)])
def test_gemm_swiglu_f16_words_for_a_q6k_down_projection(hip, dtype, m, k, n, want_fused):
    """The f16 form of the SwiGLU quants that a Q6_K down projection reads: half words of the integer
    quants, every four in the order 0, 2, 1, 3 -- whether the Q4_K epilogue writes them or the
    conversion kernel makes them from the quants afterwards (small batches, other types)."""
    _say(f"gemm_swiglu_f16 {util.NAMES[dtype]} m={m} k={k} n={n}")
    wg, _ = util.make_weights(dtype, m, k, seed=43)
    wu, _ = util.make_weights(dtype, m, k, seed=44)
    x = util.rng(m + 5 * n).standard_normal((n, k)).astype(np.float32)
    q, sc, hv, fused = hip.gemm_swiglu_f16(dtype, wg, wu, m, x, n, k)
    assert fused == want_fused
    q0, sc0, _ = hip.gemm_swiglu(dtype, wg, wu, m, x, n, k)
    assert np.array_equal(q, q0) and np.array_equal(sc.view(np.uint32), sc0.view(np.uint32))
    want = q.astype(np.float16).reshape(-1, 4)[:, [0, 2, 1, 3]].reshape(n, m)
    assert np.array_equal(hv, want.view(np.uint16))


def test_gemm_pair_refuses_mixed_types(hip):
    with pytest.raises(hip_api.HipError) as e:
        hip.gemm_pair(Q4_K, np.zeros(144 * 4, np.uint8), 4, Q6_K, np.zeros(210 * 4, np.uint8), 4,
                      np.zeros((4, 256), np.float32), 4, 256)
    assert e.value.status == 3


def test_gemm_refuses_unsupported(hip):
    with pytest.raises(hip_api.HipError) as e:  # Q5_K has no Q8_0 route: no paired / SwiGLU / block-dot entry
        hip.gemm_pair(Q5_K, np.zeros(176 * 4, np.uint8), 4, Q5_K, np.zeros(176 * 4, np.uint8), 4,
                      np.zeros((4, 256), np.float32), 4, 256)
    assert e.value.status == 3
    with pytest.raises(hip_api.HipError) as e:
        hip.gemm_block_dots(Q5_K, np.zeros(176, np.uint8), np.zeros((1, 256), np.float32), 1, 1, 256)
    assert e.value.status == 3
    with pytest.raises(hip_api.HipError) as e:  # k not a multiple of 256
        hip.gemm(Q4_0, np.zeros(18 * 4, np.uint8), np.zeros((1, 128), np.float32), 1, 1, 128)
    assert e.value.status == 3


@pytest.mark.parametrize("m,n,k,amp", [(96, 5, 1024, 1.0), (300, 77, 2048, 1.0), (130, 17, 14336, 1.0), (512, 200, 4096, 1.0),
                                         (257, 65, 512, 1e-3), (64, 130, 4096, 300.0), (1, 1, 256, 1.0), (4096, 512, 4096, 1.0)])
def test_gemm_q5k_reads_f32_activations(hip, orc, m, n, k, amp):
    """The Q5_K batched kernel dots the weights with the UNQUANTIZED activations, as cera does
    (cpu.rs:1830-1854): against the exact product in f64 the error is f32-class -- far below
    what a Q8_0 round trip of x would cost (~5e-3 rms) -- at every magnitude of x, with ragged
    tiles, a split K and a lone element; and each column agrees with the Q5_K GEMV of that token."""
    _say(f"gemm Q5_K m={m} n={n} k={k} amp={amp}")
    w, _ = util.make_weights(Q5_K, m, k, seed=41 + m)
    x = (util.rng(m + n + k).standard_normal((n, k)) * amp).astype(np.float32)
    out = hip.gemm(Q5_K, w, x, m, n, k)
    rows = np.arange(m) if m <= 600 else np.unique(np.concatenate([np.arange(8), util.rng(2).integers(0, m, 48), np.arange(m - 8, m)]))
    rb = util.H.row_bytes(Q5_K, k)
    wr = np.ascontiguousarray(w.reshape(m, rb)[rows]).reshape(-1)
    exact = util.dequant_np(Q5_K, wr, rows.size, k).astype(np.float64) @ x.astype(np.float64).T
    err = np.abs(out[rows].astype(np.float64) - exact).max()
    _say(f"  max|err|={err:.3e} rms={util.rms(exact):.3e}")
    assert err <= GEMM_TOL * util.rms(exact)
    assert err <= 3e-5 * util.rms(exact), "not f32-class: the activations were rounded somewhere"
    for j in sorted({0, n // 2, n - 1}):
        y = hip.gemv(Q5_K, wr, x[j], rows.size, k)
        assert np.abs(out[rows, j] - y).max() <= 3e-5 * util.rms(exact)


def test_gemm_q5k_lets_non_finite_activations_through(hip):
    """One NaN among a token's activations makes every output of that token NaN, as the reference's
    f32 dot does (vec_dot_q5km_f32, cera/src/backend/cpu.rs:1830-1854: NaN x weight is NaN for any
    weight) and as the Q5_K GEMV of that token does; an infinity makes them non-finite; the other
    tokens of the batch are untouched."""
    m, n, k = 96, 40, 1024
    w, _ = util.make_weights(Q5_K, m, k, seed=7)
    x = util.rng(8).standard_normal((n, k)).astype(np.float32)
    clean = hip.gemm(Q5_K, w, x, m, n, k)
    bad = x.copy()
    bad[3, 517] = np.nan
    bad[29, 0] = np.inf
    bad[31, 1023] = -np.inf
    _say("gemm Q5_K with NaN / Inf activations")
    out = hip.gemm(Q5_K, w, bad, m, n, k)
    assert np.isnan(out[:, 3]).all()
    assert not np.isfinite(out[:, 29]).any() and not np.isfinite(out[:, 31]).any()
    others = [j for j in range(n) if j not in (3, 29, 31)]
    assert np.array_equal(out[:, others].view(np.uint32), clean[:, others].view(np.uint32))
    for j in (3, 29, 31):
        y = hip.gemv(Q5_K, w, bad[j], m, k)
        assert not np.isfinite(y).any()
        if j == 3:
            assert np.isnan(y).all()   # the same NaN positions as the batched kernel: all of them


def test_q5k_model_prefills_in_batches(hip, orc):
    """A model whose Q4_K tensors are Q5_K (the Q5_K_M recipe) takes the batched prefill route:
    logits and KV cache agree with the token-by-token decode of the same prompt, and with the
    oracle's per-token forward (cera's own route for a Q5_K model, llama.rs:1643)."""
    cfg = dict(synth.TINY)
    q5 = lambda name: util.H.Q5_K if synth.q4_k_m_type(name) == util.H.Q4_K else synth.q4_k_m_type(name)
    weights = synth.make_llama(cfg, seed=91, sigma=0.05, norm_jitter=0.1, type_of=q5)
    assert weights["blk.0.attn_q.weight"][0] == util.H.Q5_K and weights["blk.0.ffn_down.weight"][0] == util.H.Q6_K
    a, b = hip_api.Model(hip, cfg, weights), hip_api.Model(hip, cfg, weights)
    om = orc.Llama(cfg, weights)
    toks = [int(t) for t in util.rng(6).integers(0, cfg["vocab"], 37)]
    _say("model: Q5_K_M batched prefill 37 tokens")
    la = a.forward_prefill(toks, 0)
    for pos, t in enumerate(toks):
        lb = b.forward(t, pos)
        lo = om.forward(t, pos)
    _say(f"  batched vs per-token cos={_cos(la, lb):.8f}; vs oracle cos={_cos(la, lo):.8f}")
    assert _cos(la, lb) > 0.999 and _cos(la, lo) > 0.999
    ka, va = a.read_kv(0)
    kb, vb = b.read_kv(0)
    assert np.abs(ka - kb).max() <= 1e-4 * util.rms(kb)   # layer 0: Q5_K k-projection of identical f32 inputs
    kl, _ = a.read_kv(cfg["n_layers"] - 1)
    kr, _ = b.read_kv(cfg["n_layers"] - 1)
    assert np.abs(kl - kr).max() <= 5e-2 * util.rms(kr)
    # all-position logits through the batched head as well
    c = hip_api.Model(hip, cfg, weights)
    allg = c.forward_prefill_logits_all(toks[:12], 0)
    assert _cos(allg[-1], hip_api.Model(hip, cfg, weights).forward_prefill(toks[:12], 0)) > 0.9999
    for mdl in (a, b, c):
        mdl.close()
    om.close()


def _cos(a, b):
    a = a.astype(np.float64); b = b.astype(np.float64)
    return float(a @ b / np.sqrt((a @ a) * (b @ b)))


def test_batched_prefill_vs_oracle(hip, orc):
    cfg = dict(synth.TINY)
    weights = synth.make_llama(cfg, seed=77, sigma=0.05, norm_jitter=0.1)
    gm = hip_api.Model(hip, cfg, weights)
    om = orc.Llama(cfg, weights)
    toks = [int(t) for t in util.rng(3).integers(0, cfg["vocab"], 40)]
    _say("model: batched prefill 40 tokens")
    lg = gm.forward_prefill(toks, 0)
    lo = om.forward_prefill_batched(toks, 0)
    assert gm.seq_len == om.seq_len == 40
    _say(f"  cos={_cos(lg, lo):.8f} max|err|={np.abs(lg - lo).max():.3e} rms={util.rms(lo):.3e}")
    assert _cos(lg, lo) > 0.999
    for layer in range(cfg["n_layers"]):
        kg, vg = gm.read_kv(layer)
        ko, vo = om.kv(layer)
        # layer 0 sees identical inputs: tight; deeper layers inherit Q8_0 rounding flips
        tol = 2e-3 if layer == 0 else 5e-2
        assert np.abs(kg - ko).max() <= tol * util.rms(ko), layer
        assert np.abs(vg - vo).max() <= tol * util.rms(vo), layer
    # a second chunk on top (start_pos > 0), then decode continues from the prefilled cache
    more = [int(t) for t in util.rng(4).integers(0, cfg["vocab"], 9)]
    lg2 = gm.forward_prefill(more, 40)
    lo2 = om.forward_prefill_batched(more, 40)
    assert _cos(lg2, lo2) > 0.999
    lg3 = gm.forward(5, 49)
    lo3 = om.forward(5, 49)
    assert _cos(lg3, lo3) > 0.999
    gm.close(); om.close()


def test_prefill_equals_decode_on_gpu(hip):
    """Batched prefill and token-by-token decode of the same prompt leave the same
    KV cache and logits (to float tolerance) -- cpu.rs:5332-5425 in spirit."""
    cfg = dict(synth.TINY)
    weights = synth.make_llama(cfg, seed=78, sigma=0.05)
    a = hip_api.Model(hip, cfg, weights)
    b = hip_api.Model(hip, cfg, weights)
    toks = [int(t) for t in util.rng(5).integers(0, cfg["vocab"], 17)]
    la = a.forward_prefill(toks, 0)
    for pos, t in enumerate(toks):
        lb = b.forward(t, pos)
    assert _cos(la, lb) > 0.999
    ka, va = a.read_kv(0)
    kb, vb = b.read_kv(0)
    assert np.abs(ka - kb).max() <= 2e-3 * util.rms(kb)
    a.close(); b.close()


@pytest.mark.parametrize("rope_type,kv_f16", [(1, False), (0, False), (1, True)])
def test_prefill_where_the_norm_adds_split_k_partial_sums(hip, orc, rope_type, kv_f16):
    """Projections whose K is split (2048-wide rows, few row tiles) in a pass of 128 tokens or more: the O
    and down projections leave their partial sums to the row norm that follows (and the last layer's down
    projection to the reduction kernel), Q | K and V theirs to the RoPE / append kernel (both pair orders,
    f32 and f16 cache).  Logits and both layers' K/V rows track the oracle's batched prefill, and a decode
    step continues from the cache."""
    cfg = dict(synth.TINY, hidden=2048, ffn=2048, n_heads=16, n_kv_heads=4, head_dim=128, max_seq_len=192, rope_type=rope_type)
    weights = synth.make_llama(cfg, seed=81, sigma=0.03, norm_jitter=0.1)
    gm = hip_api.Model(hip, cfg, weights)
    om = orc.Llama(cfg, weights)
    if kv_f16:
        gm.configure_kv(True); om.set_kv_f16(True)
    toks = [int(t) for t in util.rng(12).integers(0, cfg["vocab"], 130)]
    _say("model: 130-token prefill, hidden 2048 (split-K O and down projections)")
    lg = gm.forward_prefill(toks, 0)
    lo = om.forward_prefill_batched(toks, 0)
    _say(f"  cos={_cos(lg, lo):.8f} max|err|={np.abs(lg - lo).max():.3e} rms={util.rms(lo):.3e}")
    assert _cos(lg, lo) > 0.999
    for layer in range(cfg["n_layers"]):
        kg, vg = gm.read_kv(layer)
        ko, vo = om.kv(layer)
        tol = 2e-3 if layer == 0 else 5e-2
        assert np.abs(kg - ko).max() <= tol * util.rms(ko), layer
        assert np.abs(vg - vo).max() <= tol * util.rms(vo), layer
    lg2 = gm.forward(7, 130)
    lo2 = om.forward(7, 130)
    assert _cos(lg2, lo2) > 0.999
    gm.close(); om.close()


@pytest.mark.parametrize("nh,nkv,start,n", [(32, 8, 0, 512), (8, 2, 0, 40), (8, 8, 300, 100), (16, 2, 1000, 33),
                                             (4, 1, 0, 16), (32, 8, 4000, 96), (32, 8, 2048, 2048)])
def test_attn_prefill_batch_vs_oracle(hip, orc, nh, nkv, start, n):
    """Causal attention of a batch of queries (the tiled MFMA kernel) against the oracle's
    decode_attention evaluated query by query: query i sees positions 0 .. start + i."""
    hd = 128
    _say(f"attn_prefill nh={nh} nkv={nkv} start={start} n={n}")
    r = util.rng(7 * n + start)
    L = start + n
    q = r.standard_normal((n, nh * hd), dtype=np.float32)
    k = r.standard_normal(L * nkv * hd, dtype=np.float32)
    v = r.standard_normal(L * nkv * hd, dtype=np.float32)
    scale = 1.0 / np.sqrt(hd)
    out = hip.attn_prefill(q, k, v, nh, nkv, hd, start, n, scale)
    picks = sorted(set([0, 1, 15, 16, 31, 32, n // 2, n - 2, n - 1]) & set(range(n)))
    for i in picks:
        Li = start + i + 1
        ref = orc.decode_attention(q[i], k[:Li * nkv * hd], v[:Li * nkv * hd], nh, nkv, hd, scale, Li)
        err = np.abs(out[i].astype(np.float64) - ref).max()
        assert err <= 2e-3 * util.rms(ref), (i, err, util.rms(ref))
    assert np.isfinite(out).all()


@pytest.mark.parametrize("case", ["plain", "wide_range", "sink"])
def test_attn_prefill_split_f16_keeps_f32_accuracy(hip, orc, case):
    """The batch kernel multiplies on the f16 matrix cores with every operand split into an f16
    high and low part.  Its error against the f32 reference must stay at f32 level (far inside
    the 2e-3 bar a plain f16 product would only just meet), also when the operands span many
    binades and when the weights are one dominant key (an attention sink) plus thousands of
    keys at 1e-4 of it, where f16 alone would round the small weights coarsely."""
    nh, nkv, hd, start, n = 8, 2, 128, 3000, 64
    _say(f"attn_prefill split-f16 accuracy case={case}")
    r = util.rng(1234)
    L = start + n
    q = r.standard_normal((n, nh * hd), dtype=np.float32)
    k = r.standard_normal((L, nkv * hd), dtype=np.float32)
    v = r.standard_normal((L, nkv * hd), dtype=np.float32)
    if case == "wide_range":
        # per-dimension magnitudes from 2^-12 to 2^6: f16 subnormal low parts and large values
        mag = np.exp2(r.integers(-12, 7, hd)).astype(np.float32)
        k *= np.tile(mag, nkv); q /= np.tile(mag, nh); v *= np.tile(mag[::-1], nkv)
    if case == "sink":
        # key 0 lines up with every query: one weight of 1 against thousands near exp(-9)
        k *= 0.05
        k[0] = 0.0
        k[0, ::hd] = 60.0          # dim 0 of every KV head
        q[:, ::hd] = np.abs(q[:, ::hd]) + 2.0
    scale = 1.0 / np.sqrt(hd)
    out = hip.attn_prefill(q, k.reshape(-1), v.reshape(-1), nh, nkv, hd, start, n, scale)
    worst = 0.0
    for i in (0, 31, 32, n - 1):
        Li = start + i + 1
        ref = orc.decode_attention(q[i], k[:Li].reshape(-1), v[:Li].reshape(-1), nh, nkv, hd, scale, Li)
        worst = max(worst, np.abs(out[i].astype(np.float64) - ref).max() / util.rms(ref))
    _say(f"  max|err| / rms = {worst:.3e}")
    assert worst <= 5e-5


@pytest.mark.parametrize("kv_f16", [False, True])
@pytest.mark.parametrize("nh,nkv,start,n", [(32, 8, 0, 200), (8, 2, 300, 40), (4, 4, 1000, 33)])
def test_attn_prefill_batch_head_dim_64(hip, orc, kv_f16, nh, nkv, start, n):
    hd = 64
    _say(f"attn_prefill hd=64 nh={nh} nkv={nkv} start={start} n={n} f16={kv_f16}")
    r = util.rng(13 * n + start)
    L = start + n
    q = r.standard_normal((n, nh * hd), dtype=np.float32)
    k = r.standard_normal(L * nkv * hd, dtype=np.float32)
    v = r.standard_normal(L * nkv * hd, dtype=np.float32)
    scale = 1.0 / np.sqrt(hd)
    if kv_f16:
        out = hip.attn_f16kv(q, k, v, nh, nkv, hd, start, n, scale)
        k = k.astype(np.float16).astype(np.float32); v = v.astype(np.float16).astype(np.float32)
    else:
        out = hip.attn_prefill(q, k, v, nh, nkv, hd, start, n, scale)
    for i in sorted(set([0, 1, 31, 32, n // 2, n - 1]) & set(range(n))):
        Li = start + i + 1
        ref = orc.decode_attention(q[i], k[:Li * nkv * hd], v[:Li * nkv * hd], nh, nkv, hd, scale, Li)
        err = np.abs(out[i].astype(np.float64) - ref).max()
        assert err <= 2e-3 * util.rms(ref), (i, err, util.rms(ref))


def test_prefill_longer_than_one_pass(hip, orc):
    """A prompt beyond the 2048-token pass size is cut into passes; logits and the cache rows on
    both sides of the cut track the oracle's single batched prefill."""
    cfg = dict(synth.TINY, max_seq_len=2200)
    weights = synth.make_llama(cfg, seed=79, sigma=0.05, norm_jitter=0.1)
    gm = hip_api.Model(hip, cfg, weights)
    om = orc.Llama(cfg, weights)
    toks = [int(t) for t in util.rng(9).integers(0, cfg["vocab"], 2100)]
    _say("model: prefill 2100 tokens (two passes)")
    lg = gm.forward_prefill(toks, 0)
    lo = om.forward_prefill_batched(toks, 0)
    assert gm.seq_len == om.seq_len == 2100
    assert _cos(lg, lo) > 0.999
    kvd = cfg["n_kv_heads"] * cfg["head_dim"]
    kg, vg = gm.read_kv(0)
    ko, vo = om.kv(0)
    rows = slice(2040 * kvd, 2060 * kvd)
    assert np.abs(kg[rows] - ko[rows]).max() <= 2e-3 * util.rms(ko[rows])
    assert np.abs(vg[rows] - vo[rows]).max() <= 2e-3 * util.rms(vo[rows])
    lg2, lo2 = gm.forward(3, 2100), om.forward(3, 2100)
    assert _cos(lg2, lo2) > 0.999
    gm.close(); om.close()


@pytest.mark.parametrize("n", [5, 40])
def test_batched_prefill_when_k_is_not_a_multiple_of_256(hip, orc, n):
    """Small models' hidden sizes (896, 1536 ...) have no int8-GEMM form; their Q4_0 / Q8_0 matrices
    still take a batch through the multi-token GEMV (8 tokens per weight pass) instead of one decode
    step per token.  hidden 288, ffn 480: every K is a multiple of 32 only."""
    cfg = dict(synth.TINY, hidden=288, ffn=480, n_heads=4, n_kv_heads=2, head_dim=64)
    type_of = lambda name: Q8_0 if ("attn_v" in name or "ffn_down" in name or "token_embd" in name) else Q4_0
    weights = synth.make_llama(cfg, seed=83, sigma=0.05, type_of=type_of, norm_jitter=0.1)
    gm = hip_api.Model(hip, cfg, weights)
    om = orc.Llama(cfg, weights)
    toks = [int(t) for t in util.rng(19 + n).integers(0, cfg["vocab"], n)]
    _say(f"model: hidden 288, batched prefill of {n} tokens over Q4_0 / Q8_0")
    lg = gm.forward_prefill(toks, 0)
    lo = om.forward_prefill_per_token(toks, 0)
    assert gm.seq_len == om.seq_len == n
    assert _cos(lg, lo) > 0.999
    kg, vg = gm.read_kv(1)
    ko, vo = om.kv(1)
    assert np.abs(kg - ko).max() <= 5e-2 * util.rms(ko) and np.abs(vg - vo).max() <= 5e-2 * util.rms(vo)
    rows = gm.forward_prefill_logits_all([3, 4, 5], n)
    for i, t in enumerate([3, 4, 5]):
        assert _cos(rows[i], om.forward(t, n + i)) > 0.999, i
    gm.close(); om.close()


# ---- config 3 at the shapes the benchmark times ---------------------------------------------------
def _row_sample_check(hip, orc, dtype, w, m, k, x, n, rows):
    out = hip.gemm(dtype, w, x, m, n, k)
    rb = util.H.row_bytes(dtype, k)
    wr = np.ascontiguousarray(w.reshape(m, rb)[rows]).reshape(-1)
    ref = _oracle_gemm(orc, dtype, wr, x, rows.size, n, k)
    err = np.abs(out[rows].astype(np.float64) - ref).max()
    assert err <= GEMM_TOL * util.rms(ref), (err, util.rms(ref))
    return out


@pytest.mark.parametrize("dtype,m,k", [(Q4_K, 14336, 4096), (Q4_K, 6144, 4096)])
@pytest.mark.parametrize("n", [128, 512, 2048])
def test_gemm_config3_gate_and_qkv_shapes(hip, orc, dtype, m, k, n):
    """The gate/up projection (the shape the benchmark times) and the fused QKV height."""
    _say(f"gemm config 3 {util.NAMES[dtype]} m={m} n={n} k={k}")
    w, _ = util.make_weights(dtype, m, k, seed=11)
    x = util.rng(n + 1).standard_normal((n, k)).astype(np.float32)
    rows = np.unique(np.concatenate([np.arange(8), util.rng(2).integers(0, m, 48), np.arange(m - 8, m)]))
    _row_sample_check(hip, orc, dtype, w, m, k, x, n, rows)


@pytest.fixture(scope="module")
def head_q6k():
    m, k = 128256, 4096
    w, _ = util.make_weights(Q6_K, m, k, seed=12)
    return w, m, k


@pytest.mark.parametrize("n", [128, 512, 2048])
def test_gemm_config3_vocabulary_head(hip, orc, head_q6k, n):
    """The Q6_K output head 128256 x 4096 (the all-position logits GEMM), row-sampled."""
    w, m, k = head_q6k
    _say(f"gemm config 3 Q6_K head m={m} n={n} k={k}")
    x = util.rng(n + 2).standard_normal((n, k)).astype(np.float32)
    rows = np.unique(np.concatenate([np.arange(4), util.rng(3).integers(0, m, 40), np.arange(m - 4, m)]))
    _row_sample_check(hip, orc, Q6_K, w, m, k, x, n, rows)


@pytest.mark.parametrize("n", [128, 512, 2048])
def test_gemm_swiglu_at_ffn_shape_against_the_oracle(hip, orc, n):
    """The prefill pass's fused gate | up | SwiGLU | Q8_0 launch at 14336 x 4096, against the
    oracle's own chain gemm_preq -> silu_mul_inplace -> quantize_columns (transformer.rs:710-788,
    cpu.rs:2570-2575, transformer.rs:865-946) on a sample of 32-row quantization blocks.  The GEMM
    outputs agree with the oracle's to the float bar only, so a value that sits on a rounding
    boundary may land one int8 step away and a block maximum may round to the neighbouring f16
    scale: the dequantized result must meet the oracle's SwiGLU output within one quantization
    step, codes may differ by at most one step and only rarely, scales by at most one f16 ulp."""
    m, k = 14336, 4096
    _say(f"gemm_swiglu 14336x4096 vs oracle n={n}")
    wg, _ = util.make_weights(Q4_K, m, k, seed=51)
    wu, _ = util.make_weights(Q4_K, m, k, seed=52)
    x = util.rng(53 + n).standard_normal((n, k)).astype(np.float32)
    q, sc, fused = hip.gemm_swiglu(Q4_K, wg, wu, m, x, n, k)
    assert fused == (n >= 512), "small batches take the pair + SwiGLU kernels, large ones the fused launch"
    blocks = np.unique(np.concatenate([[0, 1, m // 32 - 1], util.rng(4).integers(0, m // 32, 5)]))
    rows = (blocks[:, None] * 32 + np.arange(32)[None, :]).reshape(-1)
    rb = util.H.row_bytes(Q4_K, k)
    g = _oracle_gemm(orc, Q4_K, np.ascontiguousarray(wg.reshape(m, rb)[rows]).reshape(-1), x, rows.size, n, k)
    u = _oracle_gemm(orc, Q4_K, np.ascontiguousarray(wu.reshape(m, rb)[rows]).reshape(-1), x, rows.size, n, k)
    h = orc.silu_mul(np.ascontiguousarray(g.T).reshape(-1), np.ascontiguousarray(u.T).reshape(-1)).reshape(n, rows.size)
    rs, rq = orc.quantize_q8_0(h.reshape(-1))
    rs, rq = rs.reshape(n, blocks.size), rq.reshape(n, rows.size)
    gq, gs = q[:, rows], sc[:, blocks]
    dq = np.abs(gq.astype(np.int32) - rq.astype(np.int32))
    assert dq.max() <= 1, int(dq.max())
    assert np.count_nonzero(dq) <= 0.02 * dq.size, np.count_nonzero(dq) / dq.size
    ulp = np.abs(gs.astype(np.float16).view(np.int16).astype(np.int32) - rs.astype(np.float16).view(np.int16).astype(np.int32))
    assert np.array_equal(gs, gs.astype(np.float16).astype(np.float32)) and ulp.max() <= 1
    deq = gq.astype(np.float32).reshape(n, blocks.size, 32) * gs[:, :, None]
    step = rs[:, :, None]
    assert (np.abs(deq - h.reshape(n, blocks.size, 32)) <= 1.01 * step + 1e-9).all()


# ---- the GEMM's integer block dots, and the route an x86 host really runs ------------------------
@pytest.mark.parametrize("dtype", util.INT8_TYPES)
@pytest.mark.parametrize("m,n,k", [(130, 70, 512), (64, 33, 1024), (9, 1, 256), (200, 5, 2048)])
def test_gemm_integer_block_dots_bit_exact(hip, orc, dtype, m, n, k):
    """Every (row, token, block) integer dot the matrix cores produce inside the prefill GEMM equals
    the brute-force integer reference (the quantities of simd.rs:6609-6629): int32 tiles of the
    int8 MFMA for Q4_0 / Q8_0 / Q4_1 / Q4_K, and for Q6_K the f32 results of the f16 MFMA, one per
    16-element scale group, which must be exact integers sum (q - 32) a."""
    _say(f"gemm block dots {util.NAMES[dtype]} m={m} n={n} k={k}")
    w, _ = util.make_weights(dtype, m, k, seed=dtype + m)
    x = util.rng(n + k).standard_normal((n, k)).astype(np.float32) * np.float32(3.0)
    dots, out = hip.gemm_block_dots(dtype, w, x, m, n, k)
    for j in range(n):
        _, xq = orc.quantize_q8_0(x[j])
        ref, asums = orc.block_dots(dtype, w, m, k, xq)
        if dtype == Q6_K:
            want = (ref - 32 * asums[None, :]).astype(np.float32)     # the kernel recentres the codes
            assert np.array_equal(dots[:, j, :], want), j
        else:
            assert np.array_equal(dots[:, j, :], ref), j
    ref_out = _oracle_gemm(orc, dtype, w, x, m, n, k)
    assert np.abs(out.astype(np.float64) - ref_out).max() <= GEMM_TOL * util.rms(ref_out)


@pytest.mark.parametrize("dtype,m,k,n", [(Q4_K, 14336, 4096, 512), (Q4_K, 4096, 4096, 128), (Q4_K, 6144, 4096, 2048),
                                         (Q4_0, 4096, 4096, 512)])
def test_gemm_against_the_x86_repacked_route(hip, orc, dtype, m, k, n):
    """cera on an x86 host multiplies repacked Q4_0 / Q4_K weights with the 8-row-interleaved
    kernels (gemm_q4_k_8x8_q8_0, cera/src/backend/simd.rs:5392-5518), not the standard-layout
    ones: the HIP GEMM meets the float bar against that route too (whole 8-row super-rows sampled)."""
    _say(f"gemm vs x86 8x8 route {util.NAMES[dtype]} m={m} n={n} k={k}")
    w, _ = util.make_weights(dtype, m, k, seed=21)
    x = util.rng(n + 9).standard_normal((n, k)).astype(np.float32)
    out = hip.gemm(dtype, w, x, m, n, k)
    srs = np.unique(np.concatenate([[0, m // 8 - 1], util.rng(6).integers(0, m // 8, 6)]))
    rows = (srs[:, None] * 8 + np.arange(8)[None, :]).reshape(-1)
    rb = util.H.row_bytes(dtype, k)
    wr = np.ascontiguousarray(w.reshape(m, rb)[rows]).reshape(-1)
    bs = np.empty((n, k // 32), np.float32); bq = np.empty((n, k), np.int8)
    for j in range(n):
        bs[j], bq[j] = orc.quantize_q8_0(x[j])
    ref = orc.gemm_preq_x86(dtype, wr, bs, bq, rows.size, n, k)
    assert np.abs(out[rows].astype(np.float64) - ref).max() <= GEMM_TOL * util.rms(ref)
