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
        _lib = L
    return _lib


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
