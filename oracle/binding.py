"""ctypes binding of the CPU oracle (``oracle/libcera_oracle.so``).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, ``__graft_entry__.smoke()``
and the ``cpu_baseline`` leg of ``bench.py``.  The shipped package
(``cera_amd``) never imports this module.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent
LIB_PATH = HERE / "libcera_oracle.so"

F32, F16, Q4_0, Q4_1, Q8_0, Q4_K, Q5_K, Q6_K, BF16 = 0, 1, 2, 3, 8, 12, 13, 14, 30
DTYPE_NAMES = {F32: "F32", F16: "F16", Q4_0: "Q4_0", Q4_1: "Q4_1", Q8_0: "Q8_0",
               Q4_K: "Q4_K", Q5_K: "Q5_K", Q6_K: "Q6_K", BF16: "BF16"}
BLOCK = {F32: (1, 4), F16: (1, 2), BF16: (1, 2), Q4_0: (32, 18), Q4_1: (32, 20), Q8_0: (32, 34),
         Q4_K: (256, 144), Q5_K: (256, 176), Q6_K: (256, 210)}


def build(force: bool = False) -> Path:
    """Compile the oracle with its Makefile (g++, no GPU needed)."""
    if force:
        subprocess.run(["make", "-C", str(HERE), "clean"], check=True, capture_output=True)
    subprocess.run(["make", "-C", str(HERE), "-j8"], check=True, capture_output=True)
    return LIB_PATH


class OrcTensor(C.Structure):
    _fields_ = [("dtype", C.c_uint32), ("_pad", C.c_uint32), ("m", C.c_uint64), ("k", C.c_uint64),
                ("data", C.c_void_p)]


class OrcLlamaLayer(C.Structure):
    _fields_ = [("attn_norm", C.c_void_p), ("ffn_norm", C.c_void_p),
                ("attn_q", OrcTensor), ("attn_k", OrcTensor), ("attn_v", OrcTensor),
                ("attn_output", OrcTensor), ("ffn_gate", OrcTensor), ("ffn_up", OrcTensor),
                ("ffn_down", OrcTensor),
                ("q_bias", C.c_void_p), ("k_bias", C.c_void_p), ("v_bias", C.c_void_p),
                ("q_norm", C.c_void_p), ("k_norm", C.c_void_p)]


class OrcLlamaConfig(C.Structure):
    _fields_ = [("n_layers", C.c_uint32), ("hidden", C.c_uint32), ("ffn", C.c_uint32),
                ("n_heads", C.c_uint32), ("n_kv_heads", C.c_uint32), ("head_dim", C.c_uint32),
                ("vocab", C.c_uint32), ("max_seq_len", C.c_uint32), ("rope_type", C.c_uint32),
                ("rope_theta", C.c_float), ("rms_eps", C.c_float), ("embed_scale", C.c_float),
                ("residual_scale", C.c_float), ("attn_scale", C.c_float), ("logit_scale", C.c_float),
                ("rope_freqs", C.c_void_p)]


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        build()
    L = C.CDLL(str(LIB_PATH))
    vp, u32, u64, i32, f32 = C.c_void_p, C.c_uint32, C.c_uint64, C.c_int, C.c_float
    sig = {
        "orc_block_elems": (u32, [u32]), "orc_block_bytes": (u32, [u32]), "orc_row_bytes": (u64, [u32, u64]),
        "orc_f16_to_f32": (f32, [C.c_uint16]), "orc_f32_to_f16": (C.c_uint16, [f32]),
        "orc_bf16_to_f32": (f32, [C.c_uint16]),
        "orc_decode_q4km_scales": (None, [vp, vp, vp]),
        "orc_dequantize_row": (i32, [u32, vp, u64, vp]),
        "orc_vec_dot_row_f32": (f32, [u32, vp, vp, u64]),
        "orc_quantize_q8_0": (None, [vp, u64, vp, vp]),
        "orc_block_dots": (i32, [u32, vp, u64, u64, vp, vp, vp]),
        "orc_gemm_preq": (i32, [u32, vp, vp, vp, vp, u64, u64, u64, i32]),
        "orc_gemv": (i32, [u32, vp, vp, vp, u64, u64, i32]),
        "orc_repack_q4_0_8x8": (i32, [vp, u64, u64, vp, vp]),
        "orc_repack_q4_k_8x8": (i32, [vp, u64, u64, vp, vp, vp]),
        "orc_gemm_q4_0_8x8_q8_0": (i32, [vp, vp, vp, vp, vp, u64, u64, u64]),
        "orc_gemm_q4_k_8x8_q8_0": (i32, [vp, vp, vp, vp, vp, vp, u64, u64, u64]),
        "orc_gemm_preq_x86": (i32, [u32, vp, vp, vp, vp, u64, u64, u64, i32]),
        "orc_llama_set_x86_repack": (None, [vp, i32]),
        "orc_gemv_f64ref": (i32, [u32, vp, vp, vp, u64, u64]),
        "orc_have_avx2": (i32, []),
        "orc_pool_create": (vp, [i32]), "orc_pool_destroy": (None, [vp]), "orc_pool_threads": (i32, [vp]),
        "orc_gemv_mt": (i32, [vp, u32, vp, vp, vp, u64, u64]),
        "orc_rmsnorm": (None, [vp, vp, u64, f32]), "orc_expf": (f32, [f32]),
        "orc_silu_mul": (None, [vp, vp, u64]), "orc_softmax": (None, [vp, u64]),
        "orc_add": (None, [vp, vp, u64]),
        "orc_rope_norm": (None, [vp, vp, u64, u32, u32, u32, f32, vp]),
        "orc_rope_neox": (None, [vp, vp, u64, u32, u32, u32, f32]),
        "orc_argmax": (u32, [vp, u64]),
        "orc_attn_scores": (None, [vp, vp, vp, u64, u64, u32, f32, u64, i32]),
        "orc_attn_values": (None, [vp, vp, vp, u64, u64, u32, u64, i32]),
        "orc_decode_attention": (None, [vp, vp, vp, u32, u32, u32, f32, u64, vp, i32]),
        "orc_llama_create": (vp, [vp, vp, vp, vp, vp, i32]),
        "orc_llama_destroy": (None, [vp]), "orc_llama_set_pool": (None, [vp, vp]),
        "orc_llama_seq_len": (u32, [vp]), "orc_llama_truncate": (None, [vp, u32]),
        "orc_llama_forward": (i32, [vp, u32, u32, vp, vp]),
        "orc_llama_forward_prefill_per_token": (i32, [vp, vp, u32, u32, vp]),
        "orc_llama_forward_prefill_batched": (i32, [vp, vp, u32, u32, vp, vp]),
        "orc_flash_attention_head": (None, [vp, vp, vp, vp, u64, u64, u64, u32, f32, u64]),
        "orc_flash_attention_head_v": (None, [vp, vp, vp, vp, u64, u64, u64, u32, f32, u64, i32]),
        "orc_llama_kcache": (vp, [vp, u32]), "orc_llama_vcache": (vp, [vp, u32]),
        "orc_rope_delta_head": (None, [vp, i32, u32, f32, u32, vp]),
        "orc_llama_shift_kv": (i32, [vp, u32, u32]),
        "orc_llama_set_kv_f16": (None, [vp, i32]),
        "orc_llama_restore_kv": (i32, [vp, u32, vp, vp, u32]),
        "orc_llama_set_seq_len": (None, [vp, u32]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(L, name, None)
        if fn is None:
            continue
        fn.restype, fn.argtypes = res, args
    _lib = L
    return L


def _p(a: np.ndarray) -> int:
    assert a.flags["C_CONTIGUOUS"], "array must be C contiguous"
    return a.ctypes.data


def have_avx2() -> bool:
    """Whether the AVX2 + FMA intrinsics twins (variant 1) can run on this host."""
    return bool(lib().orc_have_avx2())


def default_variant() -> int:
    return 1 if lib().orc_have_avx2() else 0


def row_bytes(dtype: int, k: int) -> int:
    return int(lib().orc_row_bytes(dtype, k))


def f16_to_f32(bits: int) -> float:
    return float(lib().orc_f16_to_f32(bits))


def f32_to_f16(v) -> int:
    return int(lib().orc_f32_to_f16(C.c_float(v)))


def decode_q4km_scales(scales12: bytes):
    s = np.frombuffer(bytes(scales12), dtype=np.uint8).copy()
    sc, mn = np.zeros(8, np.uint8), np.zeros(8, np.uint8)
    lib().orc_decode_q4km_scales(_p(s), _p(sc), _p(mn))
    return sc, mn


def dequantize(dtype: int, w: np.ndarray, m: int, k: int) -> np.ndarray:
    """Dequantize an [m, k] matrix stored as GGUF blocks (uint8 array) to f32."""
    w = np.ascontiguousarray(w.reshape(-1).view(np.uint8))
    rb = row_bytes(dtype, k)
    assert w.size == m * rb, (w.size, m, rb)
    out = np.empty((m, k), np.float32)
    for i in range(m):
        rc = lib().orc_dequantize_row(dtype, w.ctypes.data + i * rb, k, out[i].ctypes.data)
        assert rc == 0
    return out


def quantize_q8_0(x: np.ndarray):
    x = np.ascontiguousarray(x, np.float32).reshape(-1)
    k = x.size
    scales = np.empty(k // 32, np.float32)
    quants = np.empty(k, np.int8)
    lib().orc_quantize_q8_0(_p(x), k, _p(scales), _p(quants))
    return scales, quants


def block_dots(dtype: int, w: np.ndarray, m: int, k: int, xq: np.ndarray):
    w = np.ascontiguousarray(w.reshape(-1).view(np.uint8))
    xq = np.ascontiguousarray(xq, np.int8)
    nd = k // 16 if dtype == Q6_K else k // 32
    dots = np.zeros((m, nd), np.int32)
    asums = np.zeros(nd, np.int32)
    rc = lib().orc_block_dots(dtype, _p(w), m, k, _p(xq), _p(dots), _p(asums))
    assert rc == 0, rc
    return dots, asums


def gemv(dtype: int, w: np.ndarray, x: np.ndarray, m: int, k: int, variant: int | None = None) -> np.ndarray:
    w = np.ascontiguousarray(w.reshape(-1).view(np.uint8))
    x = np.ascontiguousarray(x, np.float32)
    y = np.empty(m, np.float32)
    v = default_variant() if variant is None else variant
    rc = lib().orc_gemv(dtype, _p(w), _p(x), _p(y), m, k, v)
    assert rc == 0, rc
    return y


def gemv_f64ref(dtype: int, w: np.ndarray, x: np.ndarray, m: int, k: int) -> np.ndarray:
    w = np.ascontiguousarray(w.reshape(-1).view(np.uint8))
    x = np.ascontiguousarray(x, np.float32)
    y = np.empty(m, np.float64)
    rc = lib().orc_gemv_f64ref(dtype, _p(w), _p(x), _p(y), m, k)
    assert rc == 0, rc
    return y


def gemm_preq(dtype: int, w: np.ndarray, b_scales: np.ndarray, b_quants: np.ndarray, m: int, n: int, k: int,
              variant: int | None = None) -> np.ndarray:
    """out[m][n]; b_scales [n][k/32], b_quants [n][k]."""
    w = np.ascontiguousarray(w.reshape(-1).view(np.uint8))
    bs = np.ascontiguousarray(b_scales, np.float32)
    bq = np.ascontiguousarray(b_quants, np.int8)
    out = np.empty((m, n), np.float32)
    v = default_variant() if variant is None else variant
    rc = lib().orc_gemm_preq(dtype, _p(w), _p(bs), _p(bq), _p(out), m, n, k, v)
    assert rc == 0, rc
    return out


def gemm_preq_x86(dtype: int, w: np.ndarray, bs: np.ndarray, bq: np.ndarray, m: int, n: int, k: int,
                  variant: int | None = None) -> np.ndarray:
    """transformer::gemm_preq as an x86 host runs it: repacked 8x8 kernels for Q4_0 / Q4_K weights
    with m % 8 == 0, the standard layout otherwise.  out [m][n]."""
    w = np.ascontiguousarray(w.reshape(-1).view(np.uint8))
    bs = np.ascontiguousarray(bs, np.float32); bq = np.ascontiguousarray(bq, np.int8)
    out = np.empty((m, n), np.float32)
    v = default_variant() if variant is None else variant
    rc = lib().orc_gemm_preq_x86(dtype, _p(w), _p(bs), _p(bq), _p(out), m, n, k, v)
    assert rc == 0, rc
    return out


def repack_8x8(dtype: int, w: np.ndarray, m: int, k: int):
    """(packed, scales) for Q4_0, (packed, dsc, dmn) for Q4_K."""
    w = np.ascontiguousarray(w.reshape(-1).view(np.uint8))
    packed = np.empty((m // 8) * (k // 32) * 128, np.uint8)
    a = np.empty((m // 8) * (k // 32) * 8, np.float32)
    if dtype == Q4_0:
        assert lib().orc_repack_q4_0_8x8(_p(w), m, k, _p(packed), _p(a)) == 0
        return packed, a
    b = np.empty_like(a)
    assert lib().orc_repack_q4_k_8x8(_p(w), m, k, _p(packed), _p(a), _p(b)) == 0
    return packed, a, b


def gemm_8x8(dtype: int, repacked, bs: np.ndarray, bq: np.ndarray, m: int, n: int, k: int) -> np.ndarray:
    bs = np.ascontiguousarray(bs, np.float32); bq = np.ascontiguousarray(bq, np.int8)
    out = np.empty((m, n), np.float32)
    if dtype == Q4_0:
        rc = lib().orc_gemm_q4_0_8x8_q8_0(_p(repacked[0]), _p(repacked[1]), _p(bs), _p(bq), _p(out), m, n, k)
    else:
        rc = lib().orc_gemm_q4_k_8x8_q8_0(_p(repacked[0]), _p(repacked[1]), _p(repacked[2]), _p(bs), _p(bq), _p(out), m, n, k)
    assert rc == 0, rc
    return out


def rmsnorm(x: np.ndarray, w: np.ndarray, eps: float) -> np.ndarray:
    y = np.array(x, np.float32, copy=True).reshape(-1)
    w = np.ascontiguousarray(w, np.float32)
    lib().orc_rmsnorm(_p(y), _p(w), y.size, eps)
    return y


def expf(x: float) -> float:
    return float(lib().orc_expf(C.c_float(x)))


def silu_mul(gate: np.ndarray, up: np.ndarray) -> np.ndarray:
    g = np.array(gate, np.float32, copy=True).reshape(-1)
    u = np.ascontiguousarray(up, np.float32)
    lib().orc_silu_mul(_p(g), _p(u), g.size)
    return g


def softmax(x: np.ndarray) -> np.ndarray:
    y = np.array(x, np.float32, copy=True).reshape(-1)
    lib().orc_softmax(_p(y), y.size)
    return y


def rope(q: np.ndarray, k: np.ndarray, pos: int, n_heads: int, n_kv_heads: int, head_dim: int, base: float,
         norm: bool = True, freq_factors: np.ndarray | None = None):
    q2 = np.array(q, np.float32, copy=True).reshape(-1)
    k2 = np.array(k, np.float32, copy=True).reshape(-1)
    if norm:
        ff = None if freq_factors is None else np.ascontiguousarray(freq_factors, np.float32)
        lib().orc_rope_norm(_p(q2), _p(k2), pos, n_heads, n_kv_heads, head_dim, base,
                            None if ff is None else _p(ff))
    else:
        lib().orc_rope_neox(_p(q2), _p(k2), pos, n_heads, n_kv_heads, head_dim, base)
    return q2, k2


def rope_delta_head(head: np.ndarray, delta_pos: int, head_dim: int, base: float, norm: bool = True,
                    freq_factors: np.ndarray | None = None) -> np.ndarray:
    """apply_rope_delta_to_head / apply_rope_norm_delta_to_head on one head."""
    h = np.array(head, np.float32, copy=True).reshape(-1)
    ff = None if freq_factors is None else np.ascontiguousarray(freq_factors, np.float32)
    lib().orc_rope_delta_head(_p(h), delta_pos, head_dim, base, 1 if norm else 0, None if ff is None else _p(ff))
    return h


def argmax(logits: np.ndarray) -> int:
    l = np.ascontiguousarray(logits, np.float32)
    return int(lib().orc_argmax(_p(l) if l.size else None, l.size))


def decode_attention(q, k_cache, v_cache, n_heads, n_kv_heads, head_dim, scale, seq_len,
                     variant: int | None = None) -> np.ndarray:
    """q [n_heads*head_dim]; k_cache/v_cache time-major [seq_len][n_kv_heads*head_dim]."""
    q = np.ascontiguousarray(q, np.float32)
    kc = np.ascontiguousarray(k_cache, np.float32)
    vc = np.ascontiguousarray(v_cache, np.float32)
    out = np.empty(n_heads * head_dim, np.float32)
    v = default_variant() if variant is None else variant
    lib().orc_decode_attention(_p(q), _p(kc), _p(vc), n_heads, n_kv_heads, head_dim, scale, seq_len, _p(out), v)
    return out


def flash_attention_head(q, k_cache, v_cache, n_queries, kv_dim, kv_h_offset, head_dim, scale, start_pos, variant=None):
    """q [n_queries][head_dim] of one head; caches time-major [pos][kv_dim].  variant None: the scalar
    route; 1 / 2: flash_attention_gqa_avx2 as intrinsics / as plain C in the same order; 0 scalar."""
    q = np.ascontiguousarray(q, np.float32)
    kc = np.ascontiguousarray(k_cache, np.float32)
    vc = np.ascontiguousarray(v_cache, np.float32)
    out = np.empty((n_queries, head_dim), np.float32)
    if variant is None:
        lib().orc_flash_attention_head(_p(q), _p(kc), _p(vc), _p(out), n_queries, kv_dim, kv_h_offset, head_dim, scale,
                                       start_pos)
    else:
        lib().orc_flash_attention_head_v(_p(q), _p(kc), _p(vc), _p(out), n_queries, kv_dim, kv_h_offset, head_dim, scale,
                                         start_pos, variant)
    return out


class Pool:
    def __init__(self, n_threads: int):
        self.h = lib().orc_pool_create(n_threads)
        self.n = n_threads

    def gemv(self, dtype, w, x, m, k, y=None):
        if y is None:
            y = np.empty(m, np.float32)
        rc = lib().orc_gemv_mt(self.h, dtype, _p(w), _p(x), _p(y), m, k)
        assert rc == 0, rc
        return y

    def close(self):
        if self.h:
            lib().orc_pool_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def _tensor(dtype, m, k, arr: np.ndarray) -> OrcTensor:
    return OrcTensor(dtype, 0, m, k, arr.ctypes.data)


class Llama:
    """Oracle twin of cera's LlamaModel (decode path). ``weights`` is the dict
    produced by the synthetic model builders: name -> (dtype, m, k, uint8 array)
    for matrices and name -> float32 array for norm vectors."""

    def __init__(self, cfg: dict, weights: dict, variant: int | None = None):
        self._keep = weights
        c = OrcLlamaConfig()
        for f in ("n_layers", "hidden", "ffn", "n_heads", "n_kv_heads", "head_dim", "vocab", "max_seq_len"):
            setattr(c, f, int(cfg[f]))
        c.rope_type = int(cfg.get("rope_type", 1))
        c.rope_theta = float(cfg.get("rope_theta", 10000.0))
        c.rms_eps = float(cfg.get("rms_eps", 1e-5))
        c.embed_scale = float(cfg.get("embed_scale", 1.0))
        c.residual_scale = float(cfg.get("residual_scale", 1.0))
        c.attn_scale = float(cfg.get("attn_scale", 0.0))
        c.logit_scale = float(cfg.get("logit_scale", 1.0))
        c.rope_freqs = None
        self.cfg = cfg
        self._opt = []
        rf = weights.get("rope_freqs.weight")
        if rf is not None:
            rf = np.ascontiguousarray(rf, np.float32)
            self._opt.append(rf)
            c.rope_freqs = rf.ctypes.data
        layers = (OrcLlamaLayer * c.n_layers)()
        for i in range(c.n_layers):
            L = layers[i]
            L.attn_norm = weights[f"blk.{i}.attn_norm.weight"].ctypes.data
            L.ffn_norm = weights[f"blk.{i}.ffn_norm.weight"].ctypes.data
            for nm in ("attn_q", "attn_k", "attn_v", "attn_output", "ffn_gate", "ffn_up", "ffn_down"):
                dt, m, k, arr = weights[f"blk.{i}.{nm}.weight"]
                setattr(L, nm, _tensor(dt, m, k, arr))
            for nm, key in (("q_bias", "attn_q.bias"), ("k_bias", "attn_k.bias"), ("v_bias", "attn_v.bias"),
                            ("q_norm", "attn_q_norm.weight"), ("k_norm", "attn_k_norm.weight")):
                a = weights.get(f"blk.{i}.{key}")
                if a is not None:
                    a = np.ascontiguousarray(a, np.float32)
                    self._opt.append(a)
                setattr(L, nm, a.ctypes.data if a is not None else None)
        dt, m, k, arr = weights["token_embd.weight"]
        embd = _tensor(dt, m, k, arr)
        outp = None
        if "output.weight" in weights:
            dt, m, k, arr = weights["output.weight"]
            outp = _tensor(dt, m, k, arr)
        v = default_variant() if variant is None else variant
        self.h = lib().orc_llama_create(C.byref(c), C.byref(embd), C.byref(outp) if outp is not None else None,
                                        weights["output_norm.weight"].ctypes.data, layers, v)
        self.vocab = c.vocab
        self.hidden = c.hidden

    def set_pool(self, pool: Pool | None):
        lib().orc_llama_set_pool(self.h, pool.h if pool else None)

    @property
    def seq_len(self) -> int:
        return int(lib().orc_llama_seq_len(self.h))

    def truncate(self, n: int):
        lib().orc_llama_truncate(self.h, n)

    def set_x86_repack(self, on: bool = True):
        """Batched prefill GEMMs through the repacked 8x8 kernels where cera's x86 build uses them."""
        lib().orc_llama_set_x86_repack(self.h, 1 if on else 0)

    def set_kv_f16(self, on: bool = True):
        """KvCompression::F16: K/V rows are rounded through IEEE half when appended."""
        lib().orc_llama_set_kv_f16(self.h, 1 if on else 0)

    def shift_kv(self, n_keep: int, shift: int) -> int:
        """0, or -1 where the reference asserts."""
        return lib().orc_llama_shift_kv(self.h, n_keep, shift)

    def restore(self, layers_kv, n_pos: int):
        """layers_kv: per layer (k, v) time-major [n_pos][kv_dim]; sets seq_len."""
        for i, (k, v) in enumerate(layers_kv):
            k = np.ascontiguousarray(k, np.float32); v = np.ascontiguousarray(v, np.float32)
            assert lib().orc_llama_restore_kv(self.h, i, _p(k), _p(v), n_pos) == 0
        lib().orc_llama_set_seq_len(self.h, n_pos)

    def forward(self, token: int, pos: int, want_hidden: bool = False):
        logits = np.empty(self.vocab, np.float32)
        hid = np.empty(self.hidden, np.float32) if want_hidden else None
        rc = lib().orc_llama_forward(self.h, token, pos, _p(logits), _p(hid) if want_hidden else None)
        assert rc == 0, rc
        return (logits, hid) if want_hidden else logits

    def forward_prefill_per_token(self, tokens, start_pos: int) -> np.ndarray:
        t = np.ascontiguousarray(tokens, np.uint32)
        logits = np.empty(self.vocab, np.float32)
        rc = lib().orc_llama_forward_prefill_per_token(self.h, _p(t), t.size, start_pos, _p(logits))
        assert rc == 0, rc
        return logits

    def forward_prefill_batched(self, tokens, start_pos: int, want_hidden: bool = False):
        t = np.ascontiguousarray(tokens, np.uint32)
        logits = np.empty(self.vocab, np.float32)
        hid = np.empty((t.size, self.hidden), np.float32) if want_hidden else None
        rc = lib().orc_llama_forward_prefill_batched(self.h, _p(t), t.size, start_pos, _p(logits),
                                                     _p(hid) if want_hidden else None)
        assert rc == 0, rc
        return (logits, hid) if want_hidden else logits

    def kv(self, layer: int):
        n = self.seq_len * self.cfg["n_kv_heads"] * self.cfg["head_dim"]
        kp = lib().orc_llama_kcache(self.h, layer)
        vp = lib().orc_llama_vcache(self.h, layer)
        k = np.ctypeslib.as_array(C.cast(kp, C.POINTER(C.c_float)), shape=(n,)).copy()
        v = np.ctypeslib.as_array(C.cast(vp, C.POINTER(C.c_float)), shape=(n,)).copy()
        return k, v

    def close(self):
        if self.h:
            lib().orc_llama_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
