"""Pins the oracle's model twin (oracle/orc_llama.cpp: forward, batched prefill) against an
independent float64 forward pass of the same architecture (tests/llama_f64.py) -- the layer
graph of cera/src/model/llama.rs:468-597 and cera/src/model/transformer.rs:1313-1652.

The two sides share no code: the f64 side works on weights unpacked by the numpy
dequantizer and never quantizes an activation; the oracle runs cera's int8 path.  What is
left between them is Q8_0 activation noise (cosine ~0.9999 on these sizes), so a cosine floor
of 0.999 holds when the graph is right -- and every deliberate graph mistake in
``llama_f64.FAULTS`` drives the cosine far below it (the second half of this file shows that
the pin bites)."""
import numpy as np
import pytest

import util
from cera_amd import host_api as H, synth
from llama_f64 import LlamaF64

COS_FLOOR = 0.999


def _cos(a, b):
    a = np.asarray(a, np.float64); b = np.asarray(b, np.float64)
    return float(a @ b / np.sqrt((a @ a) * (b @ b)))


def _small(**over):
    # 3 layers, group of 2, q_dim 256; Q8_0 everywhere keeps the weight side exact and fast
    cfg = dict(n_layers=3, hidden=256, ffn=512, n_heads=4, n_kv_heads=2, head_dim=64, vocab=384, max_seq_len=32,
               rope_type=1, rope_theta=10000.0, rms_eps=1e-5)
    cfg.update(over)
    return cfg


def _weights(cfg, seed, bias=False, qk_norm=False, freqs=False, tied=False, type_of=None):
    w = dict(synth.make_llama(cfg, seed=seed, sigma=0.06, norm_jitter=0.2, tied_output=tied,
                              type_of=type_of or (lambda name: H.Q8_0)))
    r = util.rng(seed + 1000)
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


VARIANTS = {
    "llama_norm": (dict(), dict()),
    "llama3_rope_freqs": (dict(), dict(freqs=True)),
    "qwen2_neox_bias": (dict(rope_type=0), dict(bias=True)),
    "qwen3_neox_qknorm": (dict(rope_type=0, n_heads=8, n_kv_heads=2, head_dim=64), dict(qk_norm=True)),
    "granite_scalars": (dict(embed_scale=12.0, residual_scale=0.22, attn_scale=0.0078125, logit_scale=8.0), dict()),
    "tied_head_hd128": (dict(n_heads=4, n_kv_heads=1, head_dim=128), dict(tied=True)),
    "kquant_mix": (dict(n_heads=2, n_kv_heads=1, head_dim=128), dict(type_of=synth.q4_k_m_type)),
}
TOKENS = [5, 77, 301, 12, 12, 250, 9, 100, 31, 2]


def _run_f64(cfg, w, fault=None):
    m = LlamaF64(cfg, w, fault)
    return [m.forward(t, p) for p, t in enumerate(TOKENS)]


@pytest.mark.parametrize("name", list(VARIANTS))
def test_oracle_forward_matches_independent_f64_graph(orc, name):
    over, wk = VARIANTS[name]
    cfg = _small(**over)
    w = _weights(cfg, seed=11, **wk)
    ref = _run_f64(cfg, w)
    om = orc.Llama(cfg, w)
    floor = COS_FLOOR
    worst = 1.0
    for pos, tok in enumerate(TOKENS):
        lo = om.forward(tok, pos)
        c = _cos(lo, ref[pos])
        worst = min(worst, c)
        assert c >= floor, (name, pos, c)
        s = np.sort(ref[pos])
        err = float(np.abs(lo - ref[pos]).max())
        if s[-1] - s[-2] > 4 * err:       # a clear f64 winner must be the oracle's winner too
            assert int(orc.argmax(lo)) == int(np.argmax(ref[pos])), (name, pos)
    print(f"{name}: worst cosine vs f64 graph {worst:.6f}")
    om.close()


@pytest.mark.parametrize("name", ["llama_norm", "qwen2_neox_bias", "qwen3_neox_qknorm", "granite_scalars"])
def test_oracle_batched_prefill_matches_independent_f64_graph(orc, name):
    """forward_prefill_batched (llama.rs:738-1523) against the same yardstick: last-token logits
    and the K/V rows it caches (the f64 side's rotated K and unrotated V at every position)."""
    over, wk = VARIANTS[name]
    cfg = _small(**over)
    w = _weights(cfg, seed=23, **wk)
    f = LlamaF64(cfg, w)
    ref = [f.forward(t, p) for p, t in enumerate(TOKENS)]
    om = orc.Llama(cfg, w)
    lo = om.forward_prefill_batched(TOKENS, 0)
    assert _cos(lo, ref[-1]) >= COS_FLOOR, name
    for layer in range(cfg["n_layers"]):
        ko, vo = om.kv(layer)
        kf = np.stack(f.k_cache[layer]).reshape(-1)
        vf = np.stack(f.v_cache[layer]).reshape(-1)
        assert _cos(ko, kf) >= COS_FLOOR and _cos(vo, vf) >= COS_FLOOR, (name, layer)
    om.close()


# ---- the pin bites ---------------------------------------------------------------------------
# Which deliberate mistakes each variant can see (a fault that needs biases only shows on a
# model that has them, and so on).
BITES = {
    "llama_norm": ["gqa_interleaved", "drop_ffn_norm", "drop_attn_norm", "rope_on_v", "no_rope_on_k",
                   "residual_from_normed", "swap_gate_up", "rope_layout", "skip_attn_residual", "causal_off_by_one"],
    "llama3_rope_freqs": ["freq_factors_ignored"],
    "qwen2_neox_bias": ["drop_bias", "rope_layout", "gqa_interleaved"],
    "qwen3_neox_qknorm": ["drop_qk_norm", "gqa_interleaved"],
    "granite_scalars": ["drop_residual_scale", "drop_embed_scale", "logit_scale_multiplies"],
}


@pytest.mark.parametrize("name,fault", [(n, f) for n, fs in BITES.items() for f in fs])
def test_a_wrong_graph_fails_the_pin(orc, name, fault):
    """Each single graph mistake, injected on the f64 side, breaks the agreement with the
    oracle at some position: the floor above is tight enough to tell the graphs apart."""
    over, wk = VARIANTS[name]
    cfg = _small(**over)
    w = _weights(cfg, seed=11, **wk)
    bad = _run_f64(cfg, w, fault)
    om = orc.Llama(cfg, w)
    worst = 1.0
    scale_off = False
    for pos, tok in enumerate(TOKENS):
        lo = om.forward(tok, pos)
        worst = min(worst, _cos(lo, bad[pos]))
        # a pure rescaling of the logits keeps the cosine: compare magnitudes as well
        ratio = util.rms(lo) / util.rms(bad[pos])
        scale_off |= not (0.9 < ratio < 1.1)
    om.close()
    assert worst < COS_FLOOR or scale_off, (name, fault, worst)


@pytest.mark.parametrize("name", ["llama_norm", "granite_scalars"])
def test_logit_magnitude_matches_f64_graph(orc, name):
    """Cosine is blind to a global factor (logit_scale, a missing final norm): rms must agree too."""
    over, wk = VARIANTS[name]
    cfg = _small(**over)
    w = _weights(cfg, seed=11, **wk)
    ref = _run_f64(cfg, w)
    om = orc.Llama(cfg, w)
    for pos, tok in enumerate(TOKENS):
        lo = om.forward(tok, pos)
        assert abs(util.rms(lo) / util.rms(ref[pos]) - 1.0) < 0.02, (name, pos)
    om.close()
