"""The reference-order verification route: the GPU performs exactly the f32 operations of cera's
CPU AVX2 path, in its order, so results are BIT-identical to the oracle (not merely within the
float tolerance) -- kernel by kernel, and for whole models token after token.

GEMV: gemm_q4_k_q8_0 / gemm_q6_k_q8_0 at n == 1 (cera/src/backend/simd.rs:5742-5795, 6025-6093),
row_dot_q4_0 / row_dot_q8_0 (:4593-4637), gemm_q4_1_q8_0 (:5893-5976).  Attention: attn_scores /
softmax_inplace / attn_values, AVX2 tier (cera/src/backend/cpu.rs:3503-3589, 2617-2633).
rmsnorm: cera/src/backend/cpu.rs:2479-2496.  Model: LlamaModel::forward (llama.rs:468-597).

Batched prefill as an x86 host runs it (LlamaModel::forward_prefill_batched, llama.rs:738-1523):
transformer::gemm_preq with the repacked gemm_q4_k_8x8_q8_0 / gemm_q4_0_8x8_q8_0 (simd.rs:5392-5518,
5215-5366) and the tiled K-quant / strip kernels (:5796-5851, :6094-6168), flash_attention_gqa_avx2
(cpu.rs:4261-4412).
"""
import math

import numpy as np
import pytest

import util
from cera_amd import hip_api, host_api as H, synth

pytestmark = pytest.mark.gpu


def _say(msg):
    print(msg, flush=True)


def _same_bits(a, b):
    a = np.ascontiguousarray(a, np.float32).view(np.uint32)
    b = np.ascontiguousarray(b, np.float32).view(np.uint32)
    return np.array_equal(a, b)


@pytest.mark.parametrize("dtype,m,k", [
    (util.Q4_K, 96, 4096), (util.Q4_K, 37, 256), (util.Q4_K, 64, 14336), (util.Q4_K, 33, 512),
    (util.Q6_K, 96, 4096), (util.Q6_K, 64, 14336), (util.Q6_K, 5, 256),
    (util.Q4_0, 96, 4096), (util.Q4_0, 7, 96), (util.Q8_0, 64, 4096), (util.Q8_0, 3, 32),
    (util.Q4_1, 64, 4096), (util.Q4_1, 9, 128),
])
def test_gemv_reference_order_is_bit_identical(hip, orc, dtype, m, k):
    _say(f"ref-order gemv {util.NAMES[dtype]} {m}x{k}")
    w, _ = util.make_weights(dtype, m, k, seed=m + k)
    for seed, scale in ((1, 1.0), (2, 30.0), (3, 1e-3)):
        x = util.make_x(k, seed) * np.float32(scale)
        got = hip.gemv_reference_order(dtype, w, x, m, k)
        ref = orc.gemv(dtype, w, x, m, k)            # AVX2 twin where the host has it, else the lane emulation: same bits
        assert _same_bits(got, ref), (util.NAMES[dtype], m, k, seed, float(np.abs(got - ref).max()))
    # and the fast kernel agrees with it to the float bar
    fast = hip.gemv(dtype, w, x, m, k)
    assert np.abs(fast - got).max() <= 1e-3 * util.rms(got) + 1e-12


def test_gemv_reference_order_config2_rows(hip, orc):
    """Row samples of the Llama-3-8B decode shapes (config 2): down 4096x14336 Q6_K and the
    head's 4096-wide Q6_K rows, gate 14336x4096 Q4_K."""
    for dtype, m, k in ((util.Q4_K, 512, 4096), (util.Q6_K, 256, 14336), (util.Q6_K, 1024, 4096)):
        w, _ = util.make_weights(dtype, m, k, seed=17)
        x = util.make_x(k, 5)
        assert _same_bits(hip.gemv_reference_order(dtype, w, x, m, k), orc.gemv(dtype, w, x, m, k)), (dtype, m, k)


@pytest.mark.parametrize("m,k", [(96, 4096), (5, 256), (33, 1280), (64, 14336), (1, 768)])
def test_gemv_reference_order_q5_k_reads_f32_activations(hip, orc, m, k):
    """Q5_K on the reference's route is a scalar f32 dot against the UNQUANTIZED activations
    (gemv_q5km_f32 -> vec_dot_q5_k_f32_scalar, cera/src/backend/cpu.rs:1830-1854,
    cera/src/quant.rs:892-937): four sequential 32-step chains per 64-weight pair with separate
    multiplies and adds.  Same bits, at block counts that are and are not multiples of the four
    blocks a wavefront takes per pass."""
    _say(f"ref-order gemv Q5_K {m}x{k}")
    w, _ = util.make_weights(util.Q5_K, m, k, seed=m + k)
    for seed, scale in ((1, 1.0), (2, 30.0), (3, 1e-3)):
        x = util.make_x(k, seed) * np.float32(scale)
        got = hip.gemv_reference_order(util.Q5_K, w, x, m, k)
        ref = orc.gemv(util.Q5_K, w, x, m, k)
        assert _same_bits(got, ref), (m, k, seed, float(np.abs(got - ref).max()))
    fast = hip.gemv(util.Q5_K, w, x, m, k)
    assert np.abs(fast - got).max() <= 1e-4 * util.rms(got) + 1e-12


@pytest.mark.parametrize("n_heads,n_kv,hd,L", [(32, 8, 128, 1), (32, 8, 128, 7), (32, 8, 128, 300), (8, 2, 64, 33),
                                               (4, 4, 128, 1000), (8, 1, 64, 257), (2, 1, 72, 40)])
def test_attention_reference_order_is_bit_identical(hip, orc, n_heads, n_kv, hd, L):
    if not orc.lib().orc_have_avx2():
        pytest.fail("the oracle's AVX2 attention twin needs an x86-64-v3 host")
    _say(f"ref-order attention heads {n_heads}/{n_kv} hd {hd} L {L}")
    q = util.make_x(n_heads * hd, 1)
    k = util.make_x(L * n_kv * hd, 2)
    v = util.make_x(L * n_kv * hd, 3)
    scale = 1.0 / math.sqrt(hd)
    got = hip.attn_decode_reference_order(q, k, v, n_heads, n_kv, hd, L, scale)
    ref = orc.decode_attention(q, k, v, n_heads, n_kv, hd, scale, L, variant=1)
    assert _same_bits(got, ref), float(np.abs(got - ref).max())
    if hd in (64, 128) and n_heads // n_kv in (1, 2, 4, 8):
        fast = hip.attn_decode(q, k, v, n_heads, n_kv, hd, L, scale)
        assert np.abs(fast - got).max() <= 2e-3 * max(util.rms(got), 1e-6)


@pytest.mark.parametrize("n", [128, 256, 4096, 14336, 100, 4100])
def test_rmsnorm_reference_order_is_bit_identical(hip, orc, n):
    x = util.make_x(n, n) * np.float32(3.0)
    w = (1.0 + 0.1 * util.make_x(n, n + 1)).astype(np.float32)
    assert _same_bits(hip.rmsnorm_reference_order(x, w, 1e-5), orc.rmsnorm(x, w, 1e-5))


# ---- the batched prefill's kernels ---------------------------------------------------------------
@pytest.mark.parametrize("dtype,m,k,n", [
    (util.Q4_K, 96, 4096, 5), (util.Q4_K, 64, 512, 9), (util.Q4_K, 36, 512, 3),      # 36 rows: not repacked (m % 8)
    (util.Q6_K, 96, 4096, 5), (util.Q6_K, 5, 256, 4),
    (util.Q4_0, 96, 4096, 3), (util.Q4_0, 7, 96, 2), (util.Q8_0, 64, 1024, 4), (util.Q4_1, 24, 256, 3),
])
def test_gemm_reference_order_is_bit_identical(hip, orc, dtype, m, k, n):
    """Every output element carries the bits of the x86 host's batched route: the 8x8 kernels for the
    weights cera repacks at load, the tiled (one-accumulator) K-quant kernels and the strip kernels
    otherwise -- and, with the repack switched off, of the standard route for every weight."""
    w, _ = util.make_weights(dtype, m, k, seed=m + n)
    x = util.make_x(n * k, seed=k + n).reshape(n, k)
    q = [orc.quantize_q8_0(x[j]) for j in range(n)]
    bs = np.stack([a for a, _ in q]); bq = np.stack([b for _, b in q])
    _say(f"ref-order gemm {util.NAMES[dtype]} {m}x{k} x {n}")
    got = hip.gemm_reference_order(dtype, w, x, m, k, x86_repack=True)
    assert _same_bits(got, orc.gemm_preq_x86(dtype, w, bs, bq, m, n, k)), (dtype, m, k, n)
    got = hip.gemm_reference_order(dtype, w, x, m, k, x86_repack=False)
    assert _same_bits(got, orc.gemm_preq(dtype, w, bs, bq, m, n, k)), (dtype, m, k, n)


def test_gemm_reference_order_repack_changes_bits(hip, orc):
    """The two routes really are different float chains (if they were not, the test above would pin
    nothing about which one ran)."""
    m, k, n = 64, 1024, 6
    w, _ = util.make_weights(util.Q4_K, m, k, seed=3)
    x = util.make_x(n * k, seed=4).reshape(n, k)
    a = hip.gemm_reference_order(util.Q4_K, w, x, m, k, x86_repack=True)
    b = hip.gemm_reference_order(util.Q4_K, w, x, m, k, x86_repack=False)
    assert not _same_bits(a, b) and np.abs(a - b).max() <= 1e-4 * util.rms(a)


@pytest.mark.parametrize("n_heads,n_kv,hd,n,start", [(8, 2, 128, 70, 300), (4, 4, 64, 33, 0), (6, 2, 72, 9, 40)])
def test_flash_attention_reference_order_is_bit_identical(hip, orc, n_heads, n_kv, hd, n, start):
    total = start + n
    q = util.make_x(n * n_heads * hd, 1).reshape(n, n_heads, hd)
    kc = util.make_x(total * n_kv * hd, 2)
    vc = util.make_x(total * n_kv * hd, 3)
    scale = 1.0 / math.sqrt(hd)
    _say(f"ref-order flash attention {n_heads}/{n_kv}/{hd}, {n} queries from {start}")
    got = hip.flash_attn_reference_order(q, kc, vc, n_heads, n_kv, hd, start, scale).reshape(n, n_heads, hd)
    for h in range(n_heads):
        off = (h // (n_heads // n_kv)) * hd
        ref = orc.flash_attention_head(np.ascontiguousarray(q[:, h, :]), kc, vc, n, n_kv * hd, off, hd, scale, start, variant=2)
        assert _same_bits(got[:, h, :], ref), (h,)


# ---- whole models ------------------------------------------------------------------------------
def _extras(cfg, w, seed, bias=False, qk_norm=False, freqs=False):
    w = dict(w)
    r = util.rng(seed)
    q_dim, kv_dim = cfg["n_heads"] * cfg["head_dim"], cfg["n_kv_heads"] * cfg["head_dim"]
    for i in range(cfg["n_layers"]):
        if bias:
            w[f"blk.{i}.attn_q.bias"] = (r.standard_normal(q_dim) * 0.5).astype(np.float32)
            w[f"blk.{i}.attn_k.bias"] = (r.standard_normal(kv_dim) * 0.5).astype(np.float32)
            w[f"blk.{i}.attn_v.bias"] = (r.standard_normal(kv_dim) * 0.5).astype(np.float32)
        if qk_norm:
            w[f"blk.{i}.attn_q_norm.weight"] = (1.0 + 0.3 * r.standard_normal(cfg["head_dim"])).astype(np.float32)
            w[f"blk.{i}.attn_k_norm.weight"] = (1.0 + 0.3 * r.standard_normal(cfg["head_dim"])).astype(np.float32)
    if freqs:
        w["rope_freqs.weight"] = (1.0 + 0.25 * np.arange(cfg["head_dim"] // 2)).astype(np.float32)
    return w


MODELS = {
    "llama_q4_k_m": (dict(), dict(), dict()),
    "llama3_rope_freqs": (dict(), dict(), dict(freqs=True)),
    "qwen2_neox_bias": (dict(rope_type=0), dict(), dict(bias=True)),
    "qwen3_qknorm_hd64": (dict(rope_type=0, n_heads=8, n_kv_heads=2, head_dim=64), dict(), dict(qk_norm=True)),
    "granite_scalars": (dict(embed_scale=12.0, residual_scale=0.22, attn_scale=0.0078125, logit_scale=8.0), dict(), dict()),
    "tied_q8_0": (dict(), dict(type_of=lambda name: H.Q8_0, tied_output=True), dict()),
    "q4_0": (dict(), dict(type_of=lambda name: H.Q4_0), dict()),
    # the Q5_K_M recipe: Q5_K where Q4_K_M has Q4_K, f32 activations into those matrices
    "llama_q5_k_m": (dict(), dict(type_of=lambda name: H.Q5_K if synth.q4_k_m_type(name) == H.Q4_K else synth.q4_k_m_type(name)), dict()),
}


@pytest.mark.parametrize("name", list(MODELS))
def test_model_reference_order_logits_bit_identical(hip, orc, name):
    """Prefill + free-running greedy decode: every step's logits carry the oracle's bits, so the
    token streams are identical by construction (asserted anyway)."""
    over, mk, ex = MODELS[name]
    cfg = dict(synth.TINY, **over)
    weights = _extras(cfg, synth.make_llama(cfg, seed=321, sigma=0.05, norm_jitter=0.1, **mk), 7, **ex)
    gm = hip_api.Model(hip, cfg, weights)
    om = orc.Llama(cfg, weights)
    gm.set_reference_order(True)
    assert gm.reference_order
    prompt = [int(t) for t in util.rng(5).integers(0, cfg["vocab"], 9)]
    _say(f"ref-order model {name}: prefill 9 + 20 greedy")
    lg, lo = gm.forward_prefill(prompt, 0), om.forward_prefill_per_token(prompt, 0)
    for i in range(20):
        assert _same_bits(lg, lo), (name, i, float(np.abs(lg - lo).max()))
        tg, to = int(orc.argmax(lg)), int(orc.argmax(lo))
        assert tg == to
        lg, lo = gm.forward(tg, 9 + i), om.forward(to, 9 + i)
    for layer in range(cfg["n_layers"]):
        kg, vg = gm.read_kv(layer)
        ko, vo = om.kv(layer)
        assert _same_bits(kg, ko) and _same_bits(vg, vo), (name, layer)
    # forward_greedy on this route is the same stream
    gm.truncate_kv(0); om.truncate(0)
    tg = to = 11
    for pos in range(12):
        to = int(orc.argmax(om.forward(to, pos)))
        tg = gm.forward_greedy(tg, pos)
        assert tg == to, (name, pos)
    gm.close(); om.close()


@pytest.mark.parametrize("name", ["llama_q4_k_m", "qwen2_neox_bias", "qwen3_qknorm_hd64", "granite_scalars", "q4_0"])
@pytest.mark.parametrize("n_prompt", [9, 260])
def test_model_reference_order_x86_batched_prefill(hip, orc, name, n_prompt):
    """Mode 2: a prompt of more than one token goes through forward_prefill_batched in the x86 host's
    order (repacked 8x8 GEMMs; 260 tokens: the AVX2 flash attention, 9: per-token attention).  Last-row
    logits, every cache row and the greedy continuation carry the oracle's bits -- the oracle here is
    orc.Llama with set_x86_repack(True) and forward_prefill_batched."""
    over, mk, ex = MODELS[name]
    cfg = dict(synth.TINY, max_seq_len=320, **over)
    weights = _extras(cfg, synth.make_llama(cfg, seed=123, sigma=0.05, norm_jitter=0.1, **mk), 9, **ex)
    gm = hip_api.Model(hip, cfg, weights)
    om = orc.Llama(cfg, weights)
    om.set_x86_repack(True)
    gm.set_reference_order(2)
    assert gm.reference_order == 2
    prompt = [int(t) for t in util.rng(8).integers(0, cfg["vocab"], n_prompt)]
    _say(f"ref-order x86 batched prefill {name}: {n_prompt} tokens + 12 greedy")
    lg, lo = gm.forward_prefill(prompt, 0), om.forward_prefill_batched(prompt, 0)
    assert _same_bits(lg, lo), (name, float(np.abs(lg - lo).max()))
    for layer in range(cfg["n_layers"]):
        kg, vg = gm.read_kv(layer)
        ko, vo = om.kv(layer)
        assert _same_bits(kg, ko) and _same_bits(vg, vo), (name, layer)
    for i in range(12):
        tg, to = int(orc.argmax(lg)), int(orc.argmax(lo))
        assert tg == to
        lg, lo = gm.forward(tg, n_prompt + i), om.forward(to, n_prompt + i)
        assert _same_bits(lg, lo), (name, i)
    # a second batch appended behind the first (start_pos > 0)
    more = [int(t) for t in util.rng(9).integers(0, cfg["vocab"], 7)]
    pos = n_prompt + 12
    assert _same_bits(gm.forward_prefill(more, pos), om.forward_prefill_batched(more, pos))
    gm.close(); om.close()


def test_model_reference_order_x86_batched_prefill_f16_kv(hip, orc):
    cfg = dict(synth.TINY, max_seq_len=320)
    weights = synth.make_llama(cfg, seed=45, sigma=0.05, norm_jitter=0.1)
    gm = hip_api.Model(hip, cfg, weights)
    om = orc.Llama(cfg, weights)
    gm.configure_kv(True); om.set_kv_f16(True)
    om.set_x86_repack(True)
    gm.set_reference_order(2)
    prompt = [int(t) for t in util.rng(10).integers(0, cfg["vocab"], 258)]
    assert _same_bits(gm.forward_prefill(prompt, 0), om.forward_prefill_batched(prompt, 0))
    gm.close(); om.close()


def test_final_hidden_state_matches_the_oracle(hip, orc):
    """cera_hip_read_hidden: the final normed hidden state of the last forward (what the LM head
    reads).  Bit-identical to the oracle's on the reference-order route; on the default route it
    carries the re-quantization noise of the layers below and is compared by cosine."""
    cfg = dict(synth.TINY)
    weights = synth.make_llama(cfg, seed=77, sigma=0.05, norm_jitter=0.1)
    gm = hip_api.Model(hip, cfg, weights)
    om = orc.Llama(cfg, weights)
    fast = []
    tok = 4
    for pos in range(5):
        gm.forward(tok, pos)
        fast.append(gm.read_hidden())
    gm.truncate_kv(0)
    gm.set_reference_order(True)
    for pos in range(5):
        gm.forward(tok, pos)
        _, ho = om.forward(tok, pos, want_hidden=True)
        hg = gm.read_hidden()
        assert _same_bits(hg, ho), pos
        a, b = fast[pos].astype(np.float64), ho.astype(np.float64)
        assert float(a @ b / np.sqrt((a @ a) * (b @ b))) > 0.9995, pos
    gm.close(); om.close()


def test_model_reference_order_f16_kv(hip, orc):
    cfg = dict(synth.TINY)
    weights = synth.make_llama(cfg, seed=44, sigma=0.05, norm_jitter=0.1)
    gm = hip_api.Model(hip, cfg, weights)
    om = orc.Llama(cfg, weights)
    gm.configure_kv(True); om.set_kv_f16(True)
    gm.set_reference_order(True)
    tok = 3
    for pos in range(16):
        lg, lo = gm.forward(tok, pos), om.forward(tok, pos)
        assert _same_bits(lg, lo), pos
        tok = int(orc.argmax(lo))
    gm.close(); om.close()


def test_reference_order_switch_rules(hip, orc):
    cfg = dict(synth.TINY)
    weights = synth.make_llama(cfg, seed=44, sigma=0.05)
    gm = hip_api.Model(hip, cfg, weights)
    om = orc.Llama(cfg, weights)
    fast = gm.forward(7, 0)
    with pytest.raises(hip_api.HipError) as e:
        gm.set_reference_order(True)            # the cache holds a position
    assert e.value.status == 5 and not gm.reference_order
    gm.truncate_kv(0)
    gm.set_reference_order(True)
    ref = gm.forward(7, 0)
    assert _same_bits(ref, om.forward(7, 0))
    # the default route computes the same thing up to re-quantization noise
    a, b = fast.astype(np.float64), ref.astype(np.float64)
    assert float(a @ b / np.sqrt((a @ a) * (b @ b))) > 0.9995
    gm.truncate_kv(0)
    gm.set_reference_order(False)
    assert _same_bits(gm.forward(7, 0), fast)   # and is unchanged by the round trip
    gm.close(); om.close()


def test_model_with_a_q5_k_matrix_prefills_token_by_token_in_both_modes(hip, orc):
    """A layer projection the reference's batched GEMM cannot take sends its whole prefill down
    the per-token route (cera/src/model/llama.rs:762-795): with one Q5_K matrix the x86-batched
    mode gives the per-token mode's bits, which are the oracle's."""
    cfg = dict(synth.TINY)
    w5 = synth.make_llama(cfg, seed=1, sigma=0.05, type_of=lambda name: H.Q5_K if "ffn_up" in name else H.Q8_0)
    g5 = hip_api.Model(hip, cfg, w5)
    om = orc.Llama(cfg, w5)
    prompt = [int(t) for t in util.rng(6).integers(0, cfg["vocab"], 11)]
    lo = om.forward_prefill_per_token(prompt, 0)
    for mode in (1, 2):
        g5.truncate_kv(0)
        g5.set_reference_order(mode)
        assert g5.reference_order == mode
        assert _same_bits(g5.forward_prefill(prompt, 0), lo), mode
    assert _same_bits(g5.forward(3, 11), om.forward(3, 11))
    g5.close(); om.close()
