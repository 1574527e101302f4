"""Shared test helpers: seeded synthetic inputs and an independent numpy
dequantizer written from the GGUF block-format definition (used to check the
oracle, never the other way round)."""
from __future__ import annotations

import numpy as np

from cera_amd import host_api as H

Q4_0, Q4_1, Q8_0, Q4_K, Q5_K, Q6_K = H.Q4_0, H.Q4_1, H.Q8_0, H.Q4_K, H.Q5_K, H.Q6_K
INT8_TYPES = [Q4_0, Q8_0, Q4_1, Q4_K, Q6_K]
ALL_TYPES = [Q4_0, Q4_1, Q8_0, Q4_K, Q5_K, Q6_K]
NAMES = H.TYPE_NAMES


def rng(seed):
    return np.random.default_rng(seed)


def quantize_q4_1_np(x: np.ndarray) -> np.ndarray:
    """Test-data generator for Q4_1 blocks (cera ships no Q4_1 quantizer):
    d = (max - min) / 15, m = min, q = round((x - m) / d)."""
    x = np.asarray(x, np.float32).reshape(-1, 32)
    mn = x.min(axis=1)
    mx = x.max(axis=1)
    d = ((mx - mn) / 15.0).astype(np.float16)
    m = mn.astype(np.float16)
    df = d.astype(np.float32)
    inv = np.where(df != 0, 1.0 / np.where(df != 0, df, 1), 0).astype(np.float32)
    q = np.clip(np.rint((x - m.astype(np.float32)[:, None]) * inv[:, None]), 0, 15).astype(np.uint8)
    out = np.zeros((x.shape[0], 20), np.uint8)
    out[:, 0:2] = d.view(np.uint8).reshape(-1, 2)
    out[:, 2:4] = m.view(np.uint8).reshape(-1, 2)
    out[:, 4:] = q[:, :16] | (q[:, 16:] << 4)
    return out.reshape(-1)


def make_weights(dtype: int, m: int, k: int, seed: int, sigma: float = 0.02):
    """w ~ N(0, sigma) quantized to `dtype`; returns (uint8 blocks, f32 source)."""
    w = (rng(seed).standard_normal((m, k)) * sigma).astype(np.float32)
    if dtype == Q4_1:
        return quantize_q4_1_np(w), w
    return H.quantize(dtype, w), w


def make_x(k: int, seed: int) -> np.ndarray:
    return rng(seed).standard_normal(k).astype(np.float32)


# ---- independent numpy dequantizer ---------------------------------------

def _f16(buf: np.ndarray) -> np.ndarray:
    return np.ascontiguousarray(buf).view(np.float16).astype(np.float32).reshape(-1)


def _k_scales(s: np.ndarray):
    """s: [nb, 12] uint8 -> (sc [nb, 8], mn [nb, 8]) 6-bit values (ggml get_scale_min_k4)."""
    sc = np.zeros((s.shape[0], 8), np.uint8)
    mn = np.zeros((s.shape[0], 8), np.uint8)
    sc[:, :4] = s[:, 0:4] & 63
    mn[:, :4] = s[:, 4:8] & 63
    sc[:, 4:] = (s[:, 8:12] & 0xF) | ((s[:, 0:4] >> 6) << 4)
    mn[:, 4:] = (s[:, 8:12] >> 4) | ((s[:, 4:8] >> 6) << 4)
    return sc, mn


def dequant_np(dtype: int, blocks: np.ndarray, m: int, k: int) -> np.ndarray:
    e, bsz = H.BLOCK[dtype]
    b = np.ascontiguousarray(blocks).reshape(-1).view(np.uint8).reshape(-1, bsz)
    nb = b.shape[0]
    assert nb * e == m * k
    if dtype == Q4_0:
        d = _f16(b[:, 0:2])[:, None]
        q = np.concatenate([b[:, 2:] & 0xF, b[:, 2:] >> 4], axis=1).astype(np.float32) - 8.0
        out = q * d
    elif dtype == Q4_1:
        d = _f16(b[:, 0:2])[:, None]
        mm = _f16(b[:, 2:4])[:, None]
        q = np.concatenate([b[:, 4:] & 0xF, b[:, 4:] >> 4], axis=1).astype(np.float32)
        out = q * d + mm
    elif dtype == Q8_0:
        d = _f16(b[:, 0:2])[:, None]
        out = b[:, 2:].view(np.int8).astype(np.float32) * d
    elif dtype in (Q4_K, Q5_K):
        d = _f16(b[:, 0:2])[:, None]
        dmin = _f16(b[:, 2:4])[:, None]
        sc, mn = _k_scales(b[:, 4:16])
        if dtype == Q4_K:
            qs = b[:, 16:144].reshape(nb, 4, 32)
            hi_bits = np.zeros((nb, 8, 32), np.uint8)
        else:
            qh = b[:, 16:48]
            qs = b[:, 48:176].reshape(nb, 4, 32)
            hi_bits = np.stack([((qh >> s) & 1) << 4 for s in range(8)], axis=1)
        q = np.empty((nb, 8, 32), np.float32)
        q[:, 0::2, :] = (qs & 0xF)
        q[:, 1::2, :] = (qs >> 4)
        q += hi_bits
        out = (d[:, :, None] * sc.astype(np.float32)[:, :, None]) * q - (dmin[:, :, None] * mn.astype(np.float32)[:, :, None])
        out = out.reshape(nb, 256)
    elif dtype == Q6_K:
        ql = b[:, 0:128].reshape(nb, 2, 2, 32)   # [blk][half n][ql sub-half][l]
        qh = b[:, 128:192].reshape(nb, 2, 32)
        sc = b[:, 192:208].view(np.int8).astype(np.float32)  # [nb, 16]
        d = _f16(b[:, 208:210])[:, None]
        q = np.empty((nb, 2, 4, 32), np.int32)
        for t in range(4):
            nib = (ql[:, :, t & 1, :] & 0xF) if t < 2 else (ql[:, :, t & 1, :] >> 4)
            q[:, :, t, :] = nib | (((qh >> (2 * t)) & 3) << 4)
        q = (q - 32).astype(np.float32).reshape(nb, 256)
        scale = np.repeat(sc, 16, axis=1)
        out = d * scale * q
    else:
        raise ValueError(dtype)
    return out.reshape(m, k).astype(np.float32)


def unpack_ints_np(dtype: int, blocks: np.ndarray, m: int, k: int) -> np.ndarray:
    """Integer weight codes in activation order, as the int8 kernels see them:
    Q4_0 q-8, Q8_0 w, Q4_1/Q4_K q (0..15), Q6_K q (0..63, unsigned)."""
    e, bsz = H.BLOCK[dtype]
    b = np.ascontiguousarray(blocks).reshape(-1).view(np.uint8).reshape(-1, bsz)
    nb = b.shape[0]
    if dtype == Q4_0:
        q = np.concatenate([b[:, 2:] & 0xF, b[:, 2:] >> 4], axis=1).astype(np.int32) - 8
    elif dtype == Q4_1:
        q = np.concatenate([b[:, 4:] & 0xF, b[:, 4:] >> 4], axis=1).astype(np.int32)
    elif dtype == Q8_0:
        q = b[:, 2:].view(np.int8).astype(np.int32)
    elif dtype == Q4_K:
        qs = b[:, 16:144].reshape(nb, 4, 32)
        q = np.empty((nb, 8, 32), np.int32)
        q[:, 0::2, :] = qs & 0xF
        q[:, 1::2, :] = qs >> 4
    elif dtype == Q6_K:
        ql = b[:, 0:128].reshape(nb, 2, 2, 32)
        qh = b[:, 128:192].reshape(nb, 2, 32)
        q = np.empty((nb, 2, 4, 32), np.int32)
        for t in range(4):
            nib = (ql[:, :, t & 1, :] & 0xF) if t < 2 else (ql[:, :, t & 1, :] >> 4)
            q[:, :, t, :] = nib | (((qh >> (2 * t)) & 3) << 4)
    else:
        raise ValueError(dtype)
    return q.reshape(m, k)


def rms(a) -> float:
    a = np.asarray(a, np.float64)
    return float(np.sqrt(np.mean(a * a)))
