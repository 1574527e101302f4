"""An independent float64 forward pass of the dense llama-architecture graph.

Written from the architecture's mathematics (pre-norm residual blocks, grouped
query attention, rotary embeddings, SwiGLU) on weights dequantized by the numpy
unpacker in ``util.dequant_np`` -- not from the oracle's C++ and with no
activation quantization.  It is the yardstick the oracle's model twin is pinned
against: it shares no code with it, so a graph mistake in the oracle (residual
order, which vectors are rotated, the query-head -> KV-head map, a dropped norm)
shows up as a logit disagreement far above activation-quantization noise.

The graph it states (the one cera/src/model/llama.rs:468-597 and
cera/src/model/transformer.rs:1313-1652 compute):

    h   = embed[token] * embed_scale
    per layer:
        x   = rmsnorm(h, attn_norm)
        q,k,v = Wq x (+bq), Wk x (+bk), Wv x (+bv)
        q,k = per-head rmsnorm(q, q_norm), rmsnorm(k, k_norm)      (when present)
        q,k = rope(q, pos), rope(k, pos)                           (v is never rotated)
        cache k, v at pos; head h attends KV head h // (n_heads / n_kv_heads)
        a   = softmax(q.K^T * scale) V        over positions 0..pos
        h  += residual_scale * (Wo a)
        x   = rmsnorm(h, ffn_norm)
        h  += residual_scale * (Wdown (silu(Wgate x) * (Wup x)))
    logits = Wout rmsnorm(h, output_norm) / logit_scale

``fault`` switches on ONE deliberate graph mistake; the tests use it to show that
the comparison fails when the graph is wrong.
"""
from __future__ import annotations

import numpy as np

import util

FAULTS = ("gqa_interleaved", "drop_ffn_norm", "drop_attn_norm", "rope_on_v", "no_rope_on_k", "residual_from_normed",
          "swap_gate_up", "rope_layout", "skip_attn_residual", "causal_off_by_one", "drop_residual_scale",
          "drop_embed_scale", "logit_scale_multiplies", "drop_qk_norm", "drop_bias", "freq_factors_ignored")


def _rmsnorm(x, w, eps):
    return x / np.sqrt(np.mean(x * x) + eps) * w


def _rope(vec, pos, n_heads, hd, theta, rope_type, freqs):
    """rope_type 1: adjacent pairs (2i, 2i+1); 0: split halves (i, i + hd/2).  Angle of pair i is
    pos * theta^(-2i/hd), divided by freqs[i] for the adjacent-pair layout when factors are given."""
    out = vec.reshape(n_heads, hd).copy()
    half = hd // 2
    i = np.arange(half, dtype=np.float64)
    ang = pos * theta ** (-2.0 * i / hd)
    if freqs is not None and rope_type == 1:
        ang = ang / np.asarray(freqs, np.float64)
    c, s = np.cos(ang), np.sin(ang)
    if rope_type == 1:
        a, b = out[:, 0::2].copy(), out[:, 1::2].copy()
        out[:, 0::2] = a * c - b * s
        out[:, 1::2] = a * s + b * c
    else:
        a, b = out[:, :half].copy(), out[:, half:].copy()
        out[:, :half] = a * c - b * s
        out[:, half:] = a * s + b * c
    return out.reshape(-1)


class LlamaF64:
    def __init__(self, cfg: dict, weights: dict, fault: str | None = None):
        assert fault is None or fault in FAULTS, fault
        self.cfg, self.fault = cfg, fault
        self.w = {}
        for name, val in weights.items():
            if isinstance(val, tuple):
                dt, m, k, blocks = val
                self.w[name] = util.dequant_np(dt, blocks, m, k).astype(np.float64)
            else:
                self.w[name] = np.asarray(val, np.float64)
        self.k_cache = [[] for _ in range(cfg["n_layers"])]
        self.v_cache = [[] for _ in range(cfg["n_layers"])]

    def forward(self, token: int, pos: int) -> np.ndarray:
        c, w, f = self.cfg, self.w, self.fault
        nh, nkv, hd = c["n_heads"], c["n_kv_heads"], c["head_dim"]
        eps, theta, rt = c.get("rms_eps", 1e-5), c.get("rope_theta", 10000.0), c.get("rope_type", 1)
        group = nh // nkv
        scale = c.get("attn_scale", 0.0) or 1.0 / np.sqrt(hd)
        rs = 1.0 if f == "drop_residual_scale" else c.get("residual_scale", 1.0)
        freqs = None if f == "freq_factors_ignored" else w.get("rope_freqs.weight")
        if f == "rope_layout":
            rt = 1 - rt
        assert pos == len(self.k_cache[0])
        h = w["token_embd.weight"][token].copy()
        if f != "drop_embed_scale":
            h = h * c.get("embed_scale", 1.0)
        for l in range(c["n_layers"]):
            p = f"blk.{l}."
            x = h if f == "drop_attn_norm" else _rmsnorm(h, w[p + "attn_norm.weight"], eps)
            q, k, v = w[p + "attn_q.weight"] @ x, w[p + "attn_k.weight"] @ x, w[p + "attn_v.weight"] @ x
            if p + "attn_q.bias" in w and f != "drop_bias":
                q, k, v = q + w[p + "attn_q.bias"], k + w[p + "attn_k.bias"], v + w[p + "attn_v.bias"]
            if p + "attn_q_norm.weight" in w and f != "drop_qk_norm":
                q = np.concatenate([_rmsnorm(q[i * hd:(i + 1) * hd], w[p + "attn_q_norm.weight"], eps) for i in range(nh)])
                k = np.concatenate([_rmsnorm(k[i * hd:(i + 1) * hd], w[p + "attn_k_norm.weight"], eps) for i in range(nkv)])
            q = _rope(q, pos, nh, hd, theta, rt, freqs)
            if f != "no_rope_on_k":
                k = _rope(k, pos, nkv, hd, theta, rt, freqs)
            if f == "rope_on_v":
                v = _rope(v, pos, nkv, hd, theta, rt, freqs)
            self.k_cache[l].append(k.reshape(nkv, hd))
            self.v_cache[l].append(v.reshape(nkv, hd))
            n_vis = pos if (f == "causal_off_by_one" and pos > 0) else pos + 1
            K = np.stack(self.k_cache[l][:n_vis])  # [L, nkv, hd]
            V = np.stack(self.v_cache[l][:n_vis])
            a = np.empty(nh * hd)
            for i in range(nh):
                kvh = (i % nkv) if f == "gqa_interleaved" else (i // group)
                s = K[:, kvh, :] @ q[i * hd:(i + 1) * hd] * scale
                pr = np.exp(s - s.max())
                pr /= pr.sum()
                a[i * hd:(i + 1) * hd] = pr @ V[:, kvh, :]
            o = w[p + "attn_output.weight"] @ a
            if f == "residual_from_normed":
                h = x + rs * o
            elif f != "skip_attn_residual":
                h = h + rs * o
            else:
                h = rs * o
            x = h if f == "drop_ffn_norm" else _rmsnorm(h, w[p + "ffn_norm.weight"], eps)
            g, u = w[p + "ffn_gate.weight"] @ x, w[p + "ffn_up.weight"] @ x
            if f == "swap_gate_up":
                g, u = u, g
            h = h + rs * (w[p + "ffn_down.weight"] @ (g / (1.0 + np.exp(-g)) * u))
        h = _rmsnorm(h, w["output_norm.weight"], eps)
        out = w["output.weight"] if "output.weight" in w else w["token_embd.weight"]
        logits = out @ h
        ls = c.get("logit_scale", 1.0)
        return logits * ls if f == "logit_scale_multiplies" else logits / ls
