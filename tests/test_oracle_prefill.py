"""Pins the oracle's batched prefill (cera/src/model/llama.rs:738-1523) and its
flash attention (cera/src/backend/cpu.rs:4028-4241)."""
import math

import numpy as np

import util
from cera_amd import synth


def _cos(a, b):
    a = a.astype(np.float64); b = b.astype(np.float64)
    return float(a @ b / np.sqrt((a @ a) * (b @ b)))


def test_flash_matches_naive_reference_fixture(orc):
    # cpu.rs:7091-7223: 4 heads, 2 kv heads, hd 64, n=8, start_pos 4; LCG
    # seed = seed*6364136223846793005 + 1; ((seed >> 33) as i32) * 1e-9; max diff < 1e-4
    nh, nkv, hd, n, start = 4, 2, 64, 8, 4
    seed = 0xCAFEBABE
    mask = (1 << 64) - 1

    def draw(count):
        nonlocal seed
        out = np.empty(count, np.float32)
        for i in range(count):
            seed = (seed * 6364136223846793005 + 1) & mask
            v = (seed >> 33) & 0xFFFFFFFF
            if v >= 1 << 31:
                v -= 1 << 32
            out[i] = np.float32(v) * np.float32(1e-9)
        return out

    total = start + n
    q = draw(n * nh * hd).reshape(n, nh, hd)
    kc = draw(total * nkv * hd)
    vc = draw(total * nkv * hd)
    scale = 1.0 / math.sqrt(hd)
    for h in range(nh):
        off = (h // (nh // nkv)) * hd
        got = orc.flash_attention_head(q[:, h, :], kc, vc, n, nkv * hd, off, hd, scale, start)
        for j in range(n):
            L = start + j + 1
            k = kc.reshape(total, nkv * hd)[:L, off:off + hd].astype(np.float64)
            v = vc.reshape(total, nkv * hd)[:L, off:off + hd].astype(np.float64)
            s = k @ q[j, h].astype(np.float64) * scale
            p = np.exp(s - s.max()); p /= p.sum()
            assert np.abs(got[j] - p @ v).max() < 1e-4


def test_flash_equals_decode_attention_on_long_context(orc):
    nkv, hd, n, start = 2, 128, 70, 300
    total = start + n
    q = util.make_x(n * hd, 1).reshape(n, hd)
    kc = util.make_x(total * nkv * hd, 2)
    vc = util.make_x(total * nkv * hd, 3)
    scale = 1.0 / math.sqrt(hd)
    got = orc.flash_attention_head(q, kc, vc, n, nkv * hd, hd, hd, scale, start)
    for j in (0, 17, n - 1):
        L = start + j + 1
        ref = orc.decode_attention(q[j], kc[:L * nkv * hd].reshape(L, nkv, hd)[:, 1:2, :].copy(),
                                   vc[:L * nkv * hd].reshape(L, nkv, hd)[:, 1:2, :].copy(), 1, 1, hd, scale, L)
        assert np.abs(got[j] - ref).max() < 2e-6


def test_batched_prefill_matches_per_token(orc):
    """tests/llama_batched_prefill_parity.rs: batched vs per-token prefill agree
    (cosine >= 0.9999 on the int8 path; here they differ only in the K-quant
    accumulator split, so they agree far more tightly)."""
    cfg = dict(synth.TINY)
    weights = synth.make_llama(cfg, seed=5, sigma=0.05, norm_jitter=0.1)
    a = orc.Llama(cfg, weights)
    b = orc.Llama(cfg, weights)
    toks = [int(t) for t in util.rng(1).integers(0, cfg["vocab"], 12)]
    la = a.forward_prefill_per_token(toks, 0)
    lb, hid = b.forward_prefill_batched(toks, 0, want_hidden=True)
    assert a.seq_len == b.seq_len == len(toks)
    assert _cos(la, lb) > 0.9999
    for layer in range(cfg["n_layers"]):
        ka, va = a.kv(layer)
        kb, vb = b.kv(layer)
        assert np.abs(ka - kb).max() <= 5e-2 * util.rms(ka)
    # continuing with decode works from either state
    assert _cos(a.forward(7, len(toks)), b.forward(7, len(toks))) > 0.9999
    # a second chunk appended after the first (start_pos > 0)
    more = [int(t) for t in util.rng(2).integers(0, cfg["vocab"], 5)]
    l2a = a.forward_prefill_per_token(more, a.seq_len)
    l2b = b.forward_prefill_batched(more, b.seq_len)
    assert _cos(l2a, l2b) > 0.999
