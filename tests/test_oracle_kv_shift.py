"""Pins for the oracle's n_keep context shift (delta RoPE + cache drain), following the
reference's own tests: cera/tests/n_keep_shift.rs:46-90 (delta composes with a direct rotation,
delta 0 is the identity), :139-245 (NEOX shift: head cells untouched, tail K equals a fresh
rotation for the new position, V rows keep their identity), :249-330 (the NORM twin),
cera/src/backend/cpu.rs:6666-6688 (NORM composition) and :6645-6663 (frequency factors)."""
import numpy as np
import pytest

import util
from cera_amd import synth


def _rot_closed_form(head, delta, base, norm, ff=None):
    """Independent f64 rotation: pair i turns by delta * base^(-2i/hd) / ff[i]."""
    hd = head.size
    out = head.astype(np.float64).copy()
    for i in range(hd // 2):
        ang = delta * float(base) ** (-2.0 * i / hd)
        if norm and ff is not None:
            ang /= float(ff[i])
        i0, i1 = (2 * i, 2 * i + 1) if norm else (i, i + hd // 2)
        x0, x1 = float(head[i0]), float(head[i1])
        out[i0] = x0 * np.cos(ang) - x1 * np.sin(ang)
        out[i1] = x0 * np.sin(ang) + x1 * np.cos(ang)
    return out


@pytest.mark.parametrize("norm", [False, True])
def test_delta_matches_closed_form_and_pairing(orc, norm):
    """hd = 8: which elements pair up, the sign of the rotation and the frequency schedule."""
    head = np.array([0.3, -1.1, 2.0, 0.5, -0.7, 1.3, 0.9, -0.2], np.float32)
    for delta in (1, -1, 8, -13):
        got = orc.rope_delta_head(head, delta, 8, 1e6, norm=norm)
        assert np.abs(got - _rot_closed_form(head, delta, 1e6, norm)).max() < 1e-5, delta
    # undoing a rotation returns the head; a positive delta is not its own inverse
    there = orc.rope_delta_head(head, 5, 8, 1e4, norm=norm)
    back = orc.rope_delta_head(there, -5, 8, 1e4, norm=norm)
    assert np.abs(back - head).max() < 1e-5 and np.abs(there - head).max() > 0.1


def test_delta_zero_is_identity(orc):
    original = (np.arange(32) * 0.1 + 1.0).astype(np.float32)
    for norm in (False, True):
        assert np.array_equal(orc.rope_delta_head(original, 0, 32, 1e4, norm=norm), original)


def test_delta_composes_with_direct_rotation(orc):
    hd, base = 64, 1e4
    raw = (np.arange(hd) * 0.01).astype(np.float32)
    z = np.zeros(hd, np.float32)
    for norm in (False, True):
        for p_old in (0, 1, 7, 64, 2048):
            for p_new in (0, 1, 5, 63, 2000):
                k_old = orc.rope(z, raw, p_old, 1, 1, hd, base, norm=norm)[1]
                composed = orc.rope_delta_head(k_old, p_new - p_old, hd, base, norm=norm)
                direct = orc.rope(z, raw, p_new, 1, 1, hd, base, norm=norm)[1]
                assert np.abs(composed - direct).max() < 1e-3, (norm, p_old, p_new)


def test_norm_delta_divides_by_frequency_factors(orc):
    head = np.array([1.0, 0.0, 1.0, 0.0], np.float32)
    ff = np.array([2.0, 4.0], np.float32)
    got = orc.rope_delta_head(head, 1, 4, 1e4, norm=True, freq_factors=ff)
    assert np.abs(got - _rot_closed_form(head, 1, 1e4, True, ff)).max() < 1e-5
    assert abs(got[0] - np.cos(0.5)) < 1e-5 and abs(got[1] - np.sin(0.5)) < 1e-5


def rope_filled_cache(orc, cfg, seq_len, norm, ff=None):
    """The reference fixture (n_keep_shift.rs:95-134): raw K per (layer, head, dim) rotated for
    its position; V = raw + 0.001 t so a misplaced row shows."""
    hd, nkv = cfg["head_dim"], cfg["n_kv_heads"]
    layers, raws = [], []
    for layer in range(cfg["n_layers"]):
        raw = (layer + 0.1 * np.arange(nkv)[:, None] + 0.01 * np.arange(hd)[None, :]).astype(np.float32)
        k = np.empty((seq_len, nkv, hd), np.float32)
        v = np.empty((seq_len, nkv, hd), np.float32)
        for t in range(seq_len):
            for h in range(nkv):
                k[t, h] = orc.rope_delta_head(raw[h], t, hd, cfg["rope_theta"], norm=norm, freq_factors=ff)
            v[t] = raw + np.float32(0.001) * np.float32(t)
        layers.append((k.reshape(-1), v.reshape(-1)))
        raws.append(raw)
    return layers, raws


@pytest.mark.parametrize("norm,seq_len,n_keep,shift", [(False, 24, 5, 7), (True, 24, 5, 7), (True, 30, 0, 3),
                                                        (False, 16, 4, 12)])
def test_shift_preserves_head_and_rerotates_tail(orc, norm, seq_len, n_keep, shift):
    cfg = dict(synth.TINY, rope_type=1 if norm else 0)
    weights = synth.make_llama(cfg, seed=5, sigma=0.05)
    om = orc.Llama(cfg, weights)
    layers, raws = rope_filled_cache(orc, cfg, seq_len, norm)
    om.restore(layers, seq_len)
    assert om.seq_len == seq_len
    assert om.shift_kv(n_keep, shift) == 0
    new_len = seq_len - shift
    assert om.seq_len == new_len
    hd, nkv = cfg["head_dim"], cfg["n_kv_heads"]
    for layer in range(cfg["n_layers"]):
        k, v = om.kv(layer)
        k = k.reshape(new_len, nkv, hd); v = v.reshape(new_len, nkv, hd)
        k0 = layers[layer][0].reshape(seq_len, nkv, hd)
        assert np.array_equal(k[:n_keep], k0[:n_keep])          # head cells untouched
        for t_new in range(n_keep, new_len):
            for h in range(nkv):
                fresh = orc.rope_delta_head(raws[layer][h], t_new, hd, cfg["rope_theta"], norm=norm)
                assert np.abs(k[t_new, h] - fresh).max() < 1e-3, (layer, t_new, h)
            want_v = raws[layer] + np.float32(0.001) * np.float32(t_new + shift)   # row identity kept
            assert np.abs(v[t_new] - want_v).max() < 1e-6
    om.close()


def test_shift_preconditions(orc):
    cfg = dict(synth.TINY)
    om = orc.Llama(cfg, synth.make_llama(cfg, seed=5, sigma=0.05))
    layers, _ = rope_filled_cache(orc, cfg, 10, True)
    om.restore(layers, 10)
    assert om.shift_kv(3, 0) == -1          # the reference asserts shift > 0
    assert om.shift_kv(6, 5) == -1          # ... and n_keep + shift <= seq_len
    assert om.seq_len == 10
    assert om.shift_kv(5, 5) == 0 and om.seq_len == 5   # empty tail: a pure truncation of the middle
    om.close()
