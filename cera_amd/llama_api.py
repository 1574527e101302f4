"""ctypes binding of HipLlamaModel's C face (``cera_amd/lib/libcera_hip_llama.so``).

The library links against libcera_hip.so: there is no CPU fallback, and opening
a model fails with the HIP error text when no GPU is present.
"""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import _build

LLAMA_SYMBOLS = ["cera_llama_open", "cera_llama_close", "cera_llama_last_error", "cera_llama_get_config",
                 "cera_llama_seq_len", "cera_llama_gpu_memory_bytes", "cera_llama_forward",
                 "cera_llama_forward_greedy", "cera_llama_forward_prefill", "cera_llama_forward_prefill_logits_all", "cera_llama_forward_prefill_chunked",
                 "cera_llama_set_cancel", "cera_llama_truncate_kv", "cera_llama_supports_kv_shift", "cera_llama_f16_kv_supported", "cera_llama_configure_kv_compression", "cera_llama_shift_kv",
                 "cera_llama_snapshot_state", "cera_llama_snapshot_seq_len", "cera_llama_snapshot_bytes",
                 "cera_llama_restore_state", "cera_llama_snapshot_free", "cera_llama_generate_greedy",
                 "cera_llama_set_reference_order"]


class LlamaConfigC(C.Structure):
    _fields_ = [(n, C.c_uint64) for n in ("n_layers", "hidden_size", "intermediate_size", "n_heads", "n_kv_heads",
                                          "head_dim", "vocab_size", "max_seq_len")] + \
               [("rope_theta", C.c_float), ("rms_norm_eps", C.c_float), ("rope_type", C.c_uint32)]


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not _build.LLAMA_LIB.exists():
            raise RuntimeError(f"{_build.LLAMA_LIB} is not built: run cera_amd._build.build_all() first")
        L = C.CDLL(str(_build.LLAMA_LIB))
        vp, cp, u64, u32 = C.c_void_p, C.c_char_p, C.c_uint64, C.c_uint32
        sig = {
            "cera_llama_open": (vp, [cp, u64, C.c_int, cp, u64]),
            "cera_llama_close": (None, [vp]),
            "cera_llama_last_error": (cp, [vp]),
            "cera_llama_get_config": (C.c_int, [vp, C.POINTER(LlamaConfigC)]),
            "cera_llama_seq_len": (u64, [vp]),
            "cera_llama_gpu_memory_bytes": (u64, [vp]),
            "cera_llama_forward": (C.c_int, [vp, u32, u64, vp]),
            "cera_llama_forward_greedy": (C.c_int, [vp, u32, u64, C.POINTER(u32)]),
            "cera_llama_forward_prefill": (C.c_int, [vp, vp, u64, u64, vp]),
            "cera_llama_forward_prefill_logits_all": (C.c_int, [vp, vp, u64, u64, vp]),
            "cera_llama_forward_prefill_chunked": (C.c_int, [vp, vp, u64, u64, u64, C.POINTER(u64), vp]),
            "cera_llama_set_cancel": (None, [vp, C.c_int]),
            "cera_llama_truncate_kv": (C.c_int, [vp, u64]),
            "cera_llama_supports_kv_shift": (C.c_int, [vp]),
            "cera_llama_f16_kv_supported": (C.c_int, [vp]),
            "cera_llama_configure_kv_compression": (C.c_int, [vp, C.c_int]),
            "cera_llama_shift_kv": (C.c_int, [vp, u64, u64]),
            "cera_llama_snapshot_state": (vp, [vp]),
            "cera_llama_snapshot_seq_len": (u64, [vp]),
            "cera_llama_snapshot_bytes": (u64, [vp]),
            "cera_llama_restore_state": (C.c_int, [vp, vp]),
            "cera_llama_snapshot_free": (None, [vp]),
            "cera_llama_set_reference_order": (C.c_int, [vp, C.c_int]),
            "cera_llama_generate_greedy": (C.c_int, [vp, vp, u64, u64, u64, vp, C.POINTER(C.c_double),
                                                     C.POINTER(C.c_double)]),
        }
        for name, (res, args) in sig.items():
            fn = getattr(L, name)
            fn.restype, fn.argtypes = res, args
        _lib = L
    return _lib


class BackendError(RuntimeError):
    pass


class Snapshot:
    """Opaque KV snapshot (Model::snapshot_state); restorable into any model of the same shape."""

    def __init__(self, handle):
        self.h = handle

    @property
    def seq_len(self) -> int:
        return lib().cera_llama_snapshot_seq_len(self.h)

    @property
    def nbytes(self) -> int:
        return lib().cera_llama_snapshot_bytes(self.h)

    def close(self):
        if self.h:
            lib().cera_llama_snapshot_free(self.h)
            self.h = None

    def __del__(self):
        self.close()


class HipLlama:
    """One loaded model + its InferenceState (position counter) + cancel flag."""

    def __init__(self, gguf_path: str, context_size: int = 1024, device: int = 0):
        err = C.create_string_buffer(1024)
        self.h = lib().cera_llama_open(str(gguf_path).encode(), context_size, device, err, 1024)
        if not self.h:
            raise BackendError(err.value.decode())
        c = LlamaConfigC()
        lib().cera_llama_get_config(self.h, C.byref(c))
        self.config = {n: getattr(c, n) for n, _ in LlamaConfigC._fields_}
        self.vocab = int(c.vocab_size)

    def close(self):
        if getattr(self, "h", None):
            lib().cera_llama_close(self.h)
            self.h = None

    __del__ = close

    def _check(self, rc: int):
        if rc != 0:
            raise BackendError(lib().cera_llama_last_error(self.h).decode())

    @property
    def seq_len(self) -> int:
        return int(lib().cera_llama_seq_len(self.h))

    @property
    def gpu_memory_bytes(self) -> int:
        return int(lib().cera_llama_gpu_memory_bytes(self.h))

    def forward(self, token: int, pos: int) -> np.ndarray:
        out = np.empty(self.vocab, np.float32)
        self._check(lib().cera_llama_forward(self.h, token, pos, out.ctypes.data))
        return out

    def forward_greedy(self, token: int, pos: int) -> int:
        nxt = C.c_uint32()
        self._check(lib().cera_llama_forward_greedy(self.h, token, pos, C.byref(nxt)))
        return int(nxt.value)

    def forward_prefill(self, tokens, start_pos: int) -> np.ndarray:
        t = np.ascontiguousarray(tokens, np.uint32)
        out = np.empty(self.vocab, np.float32)
        self._check(lib().cera_llama_forward_prefill(self.h, t.ctypes.data if t.size else None, t.size, start_pos,
                                                     out.ctypes.data))
        return out

    def forward_prefill_logits_all(self, tokens, start_pos: int) -> np.ndarray:
        t = np.ascontiguousarray(tokens, np.uint32)
        out = np.empty((t.size, self.vocab), np.float32)
        self._check(lib().cera_llama_forward_prefill_logits_all(self.h, t.ctypes.data if t.size else None, t.size,
                                                                start_pos, out.ctypes.data))
        return out

    def set_reference_order(self, on: bool = True):
        """Verification hook: reference-order kernels (bit-identical to the CPU AVX2 path)."""
        self._check(lib().cera_llama_set_reference_order(self.h, int(on)))

    def forward_prefill_chunked(self, tokens, start_pos: int, ubatch: int):
        t = np.ascontiguousarray(tokens, np.uint32)
        out = np.full(self.vocab, np.nan, np.float32)
        consumed = C.c_uint64()
        self._check(lib().cera_llama_forward_prefill_chunked(self.h, t.ctypes.data if t.size else None, t.size,
                                                             start_pos, ubatch, C.byref(consumed), out.ctypes.data))
        return int(consumed.value), (out if consumed.value else None)

    def set_cancel(self, flag: bool):
        lib().cera_llama_set_cancel(self.h, int(flag))

    def truncate_kv(self, n: int):
        self._check(lib().cera_llama_truncate_kv(self.h, n))

    @property
    def f16_kv_supported(self) -> bool:
        return bool(lib().cera_llama_f16_kv_supported(self.h))

    def configure_kv_compression(self, f16: bool):
        self._check(lib().cera_llama_configure_kv_compression(self.h, 1 if f16 else 0))

    @property
    def supports_kv_shift(self) -> bool:
        return bool(lib().cera_llama_supports_kv_shift(self.h))

    def shift_kv(self, n_keep: int, shift: int):
        self._check(lib().cera_llama_shift_kv(self.h, n_keep, shift))

    def snapshot_state(self) -> "Snapshot":
        s = lib().cera_llama_snapshot_state(self.h)
        if not s:
            raise BackendError(lib().cera_llama_last_error(self.h).decode())
        return Snapshot(s)

    def restore_state(self, snap: "Snapshot"):
        self._check(lib().cera_llama_restore_state(self.h, snap.h))

    def generate_greedy(self, prompt, n_new: int, ubatch: int = 512):
        p = np.ascontiguousarray(prompt, np.uint32)
        out = np.empty(n_new, np.uint32)
        tp, td = C.c_double(), C.c_double()
        self._check(lib().cera_llama_generate_greedy(self.h, p.ctypes.data, p.size, n_new, ubatch, out.ctypes.data,
                                                     C.byref(tp), C.byref(td)))
        return out, tp.value, td.value
