"""ctypes binding of the CPU host library (``cera_amd/lib/libcera_host.so``)."""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import _build

F32, F16, Q4_0, Q4_1, Q8_0, Q4_K, Q5_K, Q6_K, BF16 = 0, 1, 2, 3, 8, 12, 13, 14, 30
TYPE_NAMES = {F32: "F32", F16: "F16", Q4_0: "Q4_0", Q4_1: "Q4_1", Q8_0: "Q8_0",
              Q4_K: "Q4_K", Q5_K: "Q5_K", Q6_K: "Q6_K", BF16: "BF16"}
TYPE_IDS = {v: k for k, v in TYPE_NAMES.items()}
# (elements per block, bytes per block), cera/src/quant.rs:173-293
BLOCK = {F32: (1, 4), F16: (1, 2), BF16: (1, 2), Q4_0: (32, 18), Q4_1: (32, 20), Q8_0: (32, 34),
         Q4_K: (256, 144), Q5_K: (256, 176), Q6_K: (256, 210)}

_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not _build.HOST_LIB.exists():
            _build.build_host()
        L = C.CDLL(str(_build.HOST_LIB))
        L.cera_f16_to_f32.restype, L.cera_f16_to_f32.argtypes = C.c_float, [C.c_uint16]
        L.cera_f32_to_f16.restype, L.cera_f32_to_f16.argtypes = C.c_uint16, [C.c_float]
        L.cera_tensor_bytes.restype, L.cera_tensor_bytes.argtypes = C.c_uint64, [C.c_uint32, C.c_uint64]
        L.cera_quantize.restype = C.c_int
        L.cera_quantize.argtypes = [C.c_uint32, C.c_void_p, C.c_uint64, C.c_void_p, C.c_uint64]
        L.cera_quantize_mt.restype = C.c_int
        L.cera_quantize_mt.argtypes = [C.c_uint32, C.c_void_p, C.c_uint64, C.c_void_p, C.c_uint64, C.c_int]
        _bind_gguf(L)
        _lib = L
    return _lib


class TensorInfoC(C.Structure):
    _fields_ = [("ggml_type", C.c_uint32), ("n_dims", C.c_uint32), ("dims", C.c_uint64 * 8),
                ("offset", C.c_uint64), ("size_bytes", C.c_uint64), ("data", C.c_void_p)]


class SynthConfig(C.Structure):
    _fields_ = [("architecture", C.c_char_p),
                ("n_layers", C.c_uint32), ("hidden", C.c_uint32), ("ffn", C.c_uint32), ("n_heads", C.c_uint32),
                ("n_kv_heads", C.c_uint32), ("head_dim", C.c_uint32), ("vocab", C.c_uint32),
                ("context_length", C.c_uint32),
                ("rope_theta", C.c_float), ("rms_eps", C.c_float), ("weight_sigma", C.c_float),
                ("norm_jitter", C.c_float),
                ("type_token_embd", C.c_uint32), ("type_output", C.c_uint32), ("type_attn_q", C.c_uint32),
                ("type_attn_k", C.c_uint32), ("type_attn_v", C.c_uint32), ("type_attn_output", C.c_uint32),
                ("type_ffn_gate", C.c_uint32), ("type_ffn_up", C.c_uint32), ("type_ffn_down", C.c_uint32),
                ("tied_output", C.c_uint32), ("qkv_bias", C.c_uint32), ("qk_norm", C.c_uint32)]


def _bind_gguf(L: C.CDLL) -> None:
    vp, cp, u64, u32 = C.c_void_p, C.c_char_p, C.c_uint64, C.c_uint32
    sig = {
        "cera_gguf_open": (vp, [cp, cp, u64]),
        "cera_gguf_from_bytes": (vp, [vp, u64, cp, u64]),
        "cera_gguf_close": (None, [vp]),
        "cera_gguf_get_u32": (C.c_int, [vp, cp, C.POINTER(u32)]),
        "cera_gguf_get_f32": (C.c_int, [vp, cp, C.POINTER(C.c_float)]),
        "cera_gguf_get_str": (C.c_int64, [vp, cp, cp, u64]),
        "cera_gguf_data_offset": (u64, [vp]),
        "cera_gguf_n_tensors": (u64, [vp]),
        "cera_gguf_tensor_name": (cp, [vp, u64]),
        "cera_gguf_tensor": (C.c_int, [vp, cp, C.POINTER(TensorInfoC)]),
        "cera_gguf_writer_new": (vp, [u32]),
        "cera_gguf_writer_free": (None, [vp]),
        "cera_gguf_writer_add_u32": (None, [vp, cp, u32]),
        "cera_gguf_writer_add_f32": (None, [vp, cp, C.c_float]),
        "cera_gguf_writer_add_str": (None, [vp, cp, cp]),
        "cera_gguf_writer_add_tensor": (None, [vp, cp, C.POINTER(u64), u32, u32, vp, u64]),
        "cera_gguf_writer_write": (C.c_int, [vp, cp, cp, u64]),
        "cera_synth_llama_gguf": (C.c_int, [cp, C.POINTER(SynthConfig), u64, C.c_int, cp, u64]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(L, name)
        fn.restype, fn.argtypes = res, args


HOST_SYMBOLS = ["cera_f16_to_f32", "cera_f32_to_f16", "cera_tensor_bytes", "cera_quantize", "cera_quantize_mt",
                "cera_gguf_open", "cera_gguf_from_bytes", "cera_gguf_close", "cera_gguf_get_u32", "cera_gguf_get_f32",
                "cera_gguf_get_str", "cera_gguf_data_offset", "cera_gguf_n_tensors", "cera_gguf_tensor_name",
                "cera_gguf_tensor", "cera_gguf_writer_new", "cera_gguf_writer_free", "cera_gguf_writer_add_u32",
                "cera_gguf_writer_add_f32", "cera_gguf_writer_add_str", "cera_gguf_writer_add_tensor",
                "cera_gguf_writer_write", "cera_synth_llama_gguf"]


class GgufError(RuntimeError):
    pass


class Gguf:
    """A parsed GGUF v3 file (mmap-backed) or byte buffer."""

    def __init__(self, path: str | None = None, data: bytes | None = None):
        err = C.create_string_buffer(512)
        if path is not None:
            self.h = lib().cera_gguf_open(str(path).encode(), err, 512)
        else:
            self._buf = np.frombuffer(data, np.uint8)
            self.h = lib().cera_gguf_from_bytes(self._buf.ctypes.data if self._buf.size else None, self._buf.size,
                                                err, 512)
        if not self.h:
            raise GgufError(err.value.decode())

    def close(self):
        if self.h:
            lib().cera_gguf_close(self.h)
            self.h = None

    def __enter__(self):
        return self

    def __exit__(self, *a):
        self.close()

    def get_u32(self, key: str):
        v = C.c_uint32()
        return int(v.value) if lib().cera_gguf_get_u32(self.h, key.encode(), C.byref(v)) else None

    def get_f32(self, key: str):
        v = C.c_float()
        return float(v.value) if lib().cera_gguf_get_f32(self.h, key.encode(), C.byref(v)) else None

    def get_str(self, key: str):
        n = lib().cera_gguf_get_str(self.h, key.encode(), None, 0)
        if n < 0:
            return None
        buf = C.create_string_buffer(n + 1)
        lib().cera_gguf_get_str(self.h, key.encode(), buf, n + 1)
        return buf.value.decode()

    @property
    def data_offset(self) -> int:
        return int(lib().cera_gguf_data_offset(self.h))

    def tensor_names(self) -> list[str]:
        return [lib().cera_gguf_tensor_name(self.h, i).decode() for i in range(lib().cera_gguf_n_tensors(self.h))]

    def tensor_info(self, name: str):
        t = TensorInfoC()
        if not lib().cera_gguf_tensor(self.h, name.encode(), C.byref(t)):
            return None
        return dict(ggml_type=int(t.ggml_type), dims=[int(t.dims[i]) for i in range(t.n_dims)],
                    offset=int(t.offset), size_bytes=int(t.size_bytes), data=t.data)

    def tensor_bytes(self, name: str) -> np.ndarray:
        """A copy of the tensor's payload as uint8."""
        t = self.tensor_info(name)
        if t is None or not t["size_bytes"]:
            raise KeyError(name)
        return np.ctypeslib.as_array(C.cast(t["data"], C.POINTER(C.c_uint8)), (t["size_bytes"],)).copy()

    def llama_weights(self) -> tuple[dict, dict]:
        """(cfg, weights) in the shape the model constructors of this package take:
        matrices as (ggml_type, m, k, uint8 blocks), vectors as float32 arrays."""
        arch = self.get_str("general.architecture")
        g = lambda k: self.get_u32(f"{arch}.{k}")
        cfg = dict(n_layers=g("block_count"), hidden=g("embedding_length"), ffn=g("feed_forward_length"),
                   n_heads=g("attention.head_count"), n_kv_heads=g("attention.head_count_kv"),
                   vocab=g("vocab_size"), max_seq_len=g("context_length"),
                   rope_type=0 if arch in ("qwen2", "qwen3") else 1,
                   rope_theta=self.get_f32(f"{arch}.rope.freq_base") or 1000000.0,
                   rms_eps=self.get_f32(f"{arch}.attention.layer_norm_rms_epsilon") or 1e-6)
        cfg["head_dim"] = g("attention.key_length") or cfg["hidden"] // cfg["n_heads"]
        weights = {}
        for name in self.tensor_names():
            t = self.tensor_info(name)
            raw = self.tensor_bytes(name)
            if len(t["dims"]) == 1:
                assert t["ggml_type"] == F32, name
                weights[name] = raw.view(np.float32)
            else:
                weights[name] = (t["ggml_type"], t["dims"][1], t["dims"][0], raw)
        return cfg, weights


class GgufWriter:
    def __init__(self, alignment: int = 32):
        self.h = lib().cera_gguf_writer_new(alignment)
        self._keep = []

    def add_u32(self, key: str, v: int):
        lib().cera_gguf_writer_add_u32(self.h, key.encode(), v)

    def add_f32(self, key: str, v: float):
        lib().cera_gguf_writer_add_f32(self.h, key.encode(), v)

    def add_str(self, key: str, v: str):
        lib().cera_gguf_writer_add_str(self.h, key.encode(), v.encode())

    def add_tensor(self, name: str, dims, ggml_type: int, data: np.ndarray):
        """dims in GGUF order (row length first); data: the payload bytes."""
        data = np.ascontiguousarray(data).reshape(-1).view(np.uint8)
        self._keep.append(data)
        d = (C.c_uint64 * len(dims))(*dims)
        lib().cera_gguf_writer_add_tensor(self.h, name.encode(), d, len(dims), ggml_type,
                                          data.ctypes.data if data.size else None, data.size)

    def write(self, path: str):
        err = C.create_string_buffer(512)
        if lib().cera_gguf_writer_write(self.h, str(path).encode(), err, 512) != 0:
            raise GgufError(err.value.decode())

    def __del__(self):
        if getattr(self, "h", None):
            lib().cera_gguf_writer_free(self.h)
            self.h = None


def synth_llama_gguf(path: str, cfg: dict, seed: int = 1, n_threads: int = 8, sigma: float = 0.02,
                     norm_jitter: float = 0.0, types: dict | None = None, tied_output: bool = False,
                     qkv_bias: bool = False, qk_norm: bool = False, arch: str = "llama",
                     explicit_head_dim: bool = True) -> None:
    """Write a seeded random-init llama-architecture GGUF.  ``cfg`` uses the keys of
    ``cera_amd.synth`` configs; ``types`` overrides the Q4_K_M-style per-tensor mix
    (keys: token_embd, output, attn_q, attn_k, attn_v, attn_output, ffn_gate, ffn_up, ffn_down)."""
    t = dict(token_embd=Q4_K, output=Q6_K, attn_q=Q4_K, attn_k=Q4_K, attn_v=Q6_K, attn_output=Q4_K,
             ffn_gate=Q4_K, ffn_up=Q4_K, ffn_down=Q6_K)
    t.update(types or {})
    c = SynthConfig()
    c.architecture = arch.encode()
    for f in ("n_layers", "hidden", "ffn", "n_heads", "n_kv_heads", "vocab"):
        setattr(c, f, int(cfg[f]))
    c.head_dim = int(cfg["head_dim"]) if explicit_head_dim else 0
    c.context_length = int(cfg["max_seq_len"])
    c.rope_theta, c.rms_eps = float(cfg["rope_theta"]), float(cfg["rms_eps"])
    c.weight_sigma, c.norm_jitter = sigma, norm_jitter
    for k, v in t.items():
        setattr(c, "type_" + k, v)
    c.tied_output, c.qkv_bias, c.qk_norm = int(tied_output), int(qkv_bias), int(qk_norm)
    err = C.create_string_buffer(512)
    if lib().cera_synth_llama_gguf(str(path).encode(), C.byref(c), seed, n_threads, err, 512) != 0:
        raise GgufError(err.value.decode())


def row_bytes(ggml_type: int, k: int) -> int:
    e, b = BLOCK[ggml_type]
    if k % e:
        raise ValueError(f"k={k} is not a multiple of the {TYPE_NAMES[ggml_type]} block size {e}")
    return k // e * b


def tensor_bytes(ggml_type: int, n: int) -> int:
    return int(lib().cera_tensor_bytes(ggml_type, n))


def quantize(ggml_type: int, x: np.ndarray, n_threads: int = 1) -> np.ndarray:
    """Quantize a float32 array (any shape, row-major) to GGUF blocks; returns uint8."""
    x = np.ascontiguousarray(x, np.float32).reshape(-1)
    if ggml_type == F32:
        return x.view(np.uint8).copy()
    nbytes = tensor_bytes(ggml_type, x.size)
    if nbytes == 0:
        raise ValueError(f"cannot store {x.size} elements as {TYPE_NAMES.get(ggml_type, ggml_type)}")
    out = np.empty(nbytes, np.uint8)
    rc = lib().cera_quantize_mt(ggml_type, x.ctypes.data, x.size, out.ctypes.data, nbytes, n_threads)
    if rc != 0:
        raise ValueError(f"cera_quantize failed for type {ggml_type}")
    return out
