"""Seeded synthetic llama-architecture weights (random init, GGUF tensor names).

Matrices are w ~ N(0, sigma) quantized with the GGUF quantizers of the host
library; norm vectors are 1.0.  The tensor-type mix follows the Q4_K_M-style
policy of cera/src/convert/quantize.rs:102-113 unless overridden.
"""
from __future__ import annotations

import numpy as np

from . import host_api as H

LLAMA3_8B = dict(n_layers=32, hidden=4096, ffn=14336, n_heads=32, n_kv_heads=8, head_dim=128, vocab=128256,
                 max_seq_len=1024, rope_type=1, rope_theta=500000.0, rms_eps=1e-5)

TINY = dict(n_layers=2, hidden=256, ffn=512, n_heads=4, n_kv_heads=2, head_dim=128, vocab=512,
            max_seq_len=64, rope_type=1, rope_theta=10000.0, rms_eps=1e-5)


def q4_k_m_type(name: str, embd_type: int = H.Q4_K) -> int:
    if "attn_v" in name or "ffn_down" in name or name == "output.weight":
        return H.Q6_K
    if "token_embd" in name:
        return embd_type
    return H.Q4_K


def tensor_shapes(cfg: dict, tied_output: bool = False):
    """(name, m, k) of every matrix, GGUF naming (shape on disk is [k, m])."""
    hs, ffn = cfg["hidden"], cfg["ffn"]
    q_dim = cfg["n_heads"] * cfg["head_dim"]
    kv_dim = cfg["n_kv_heads"] * cfg["head_dim"]
    out = [("token_embd.weight", cfg["vocab"], hs)]
    if not tied_output:
        out.append(("output.weight", cfg["vocab"], hs))
    for i in range(cfg["n_layers"]):
        p = f"blk.{i}."
        out += [(p + "attn_q.weight", q_dim, hs), (p + "attn_k.weight", kv_dim, hs), (p + "attn_v.weight", kv_dim, hs),
                (p + "attn_output.weight", hs, q_dim), (p + "ffn_gate.weight", ffn, hs), (p + "ffn_up.weight", ffn, hs),
                (p + "ffn_down.weight", hs, ffn)]
    return out


def make_llama(cfg: dict, seed: int, sigma: float = 0.02, type_of=q4_k_m_type, tied_output: bool = False,
               n_threads: int = 8, norm_jitter: float = 0.0) -> dict:
    """name -> (ggml_type, m, k, uint8 blocks) | float32 vector."""
    ss = np.random.SeedSequence(seed)
    weights = {}
    shapes = tensor_shapes(cfg, tied_output)
    for (name, m, k), child in zip(shapes, ss.spawn(len(shapes))):
        rng = np.random.default_rng(child)
        w = rng.standard_normal((m, k), dtype=np.float32)
        w *= np.float32(sigma)
        t = type_of(name)
        weights[name] = (t, m, k, H.quantize(t, w, n_threads))
    rng = np.random.default_rng(ss.spawn(1)[0])

    def norm_vec(n):
        v = np.ones(n, np.float32)
        if norm_jitter:
            v += (rng.standard_normal(n) * norm_jitter).astype(np.float32)
        return v

    weights["output_norm.weight"] = norm_vec(cfg["hidden"])
    for i in range(cfg["n_layers"]):
        weights[f"blk.{i}.attn_norm.weight"] = norm_vec(cfg["hidden"])
        weights[f"blk.{i}.ffn_norm.weight"] = norm_vec(cfg["hidden"])
    return weights
