"""A host for the LOWER ABI (include/cera_hip_kernels.h) that does not use libcera_hip.so at all:
plain ctypes on the HIP runtime -- hipMalloc / hipMemcpy / hipModuleLoad / hipModuleLaunchKernel
on the standalone code object ``cera_hip_gfx950.hsaco``.  It is what a pure-Rust ``hip-sys`` host
inside cera would do, written down as runnable code; the tests use it to show that the code
object alone reproduces the library's results bit for bit.
"""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import _build

GGML_NAMES = {2: "q4_0", 3: "q4_1", 8: "q8_0", 12: "q4_k", 14: "q6_k"}
BLOCK = {2: (32, 18), 3: (32, 20), 8: (32, 34), 12: (256, 144), 14: (256, 210)}   # elems, bytes


class QuantizeArgs(C.Structure):   # cera_k_quantize_q8_0_args
    _fields_ = [("x", C.c_void_p), ("k", C.c_uint64), ("scales", C.c_void_p), ("quants", C.c_void_p), ("bsum", C.c_void_p)]


class RmsnormQ8Args(C.Structure):  # cera_k_rmsnorm_q8_0_args
    _fields_ = [("x", C.c_void_p), ("w", C.c_void_p), ("n", C.c_uint32), ("eps", C.c_float), ("y", C.c_void_p),
                ("scales", C.c_void_p), ("quants", C.c_void_p)]


class GemvArgs(C.Structure):       # cera_k_gemv_args
    _fields_ = [("w", C.c_void_p), ("w2", C.c_void_p), ("xq", C.c_void_p), ("xs", C.c_void_p), ("y", C.c_void_p),
                ("resid", C.c_void_p), ("m", C.c_uint32), ("n_units", C.c_uint32), ("row_bytes", C.c_uint32),
                ("rows_per_group", C.c_uint32), ("dbg_dots", C.c_void_p), ("dbg_stride", C.c_uint32), ("dbg_asums", C.c_void_p)]


class HipRuntimeError(RuntimeError):
    pass


class Host:
    """Device 0, the default stream, one loaded module."""

    def __init__(self, hsaco_path: str | None = None, device: int = 0):
        self.hip = C.CDLL("libamdhip64.so")
        self.hip.hipGetErrorString.restype = C.c_char_p
        self._ck(self.hip.hipSetDevice(device), "hipSetDevice")
        self.module = C.c_void_p()
        path = str(hsaco_path or _build.HSACO)
        self._ck(self.hip.hipModuleLoad(C.byref(self.module), path.encode()), f"hipModuleLoad({path})")
        self._fns = {}
        self._bufs = []

    def _ck(self, err, what):
        if err != 0:
            raise HipRuntimeError(f"{what}: {self.hip.hipGetErrorString(err).decode()}")

    def close(self):
        for b in self._bufs:
            self.hip.hipFree(b)
        self._bufs = []
        if self.module:
            self.hip.hipModuleUnload(self.module)
            self.module = None

    def function(self, name: str):
        if name not in self._fns:
            f = C.c_void_p()
            self._ck(self.hip.hipModuleGetFunction(C.byref(f), self.module, name.encode()), f"hipModuleGetFunction({name})")
            self._fns[name] = f
        return self._fns[name]

    def malloc(self, nbytes: int) -> int:
        p = C.c_void_p()
        self._ck(self.hip.hipMalloc(C.byref(p), C.c_size_t(max(nbytes, 16))), "hipMalloc")
        self._bufs.append(p)
        return p.value

    def upload(self, arr: np.ndarray) -> int:
        arr = np.ascontiguousarray(arr)
        d = self.malloc(arr.nbytes)
        self._ck(self.hip.hipMemcpy(C.c_void_p(d), C.c_void_p(arr.ctypes.data), C.c_size_t(arr.nbytes), 1), "hipMemcpy H2D")
        return d

    def download(self, dev: int, shape, dtype) -> np.ndarray:
        out = np.empty(shape, dtype)
        self._ck(self.hip.hipDeviceSynchronize(), "hipDeviceSynchronize")
        self._ck(self.hip.hipMemcpy(C.c_void_p(out.ctypes.data), C.c_void_p(dev), C.c_size_t(out.nbytes), 2), "hipMemcpy D2H")
        return out

    def launch(self, name: str, grid: int, block: int, args: C.Structure):
        params = (C.c_void_p * 1)(C.cast(C.pointer(args), C.c_void_p))
        self._ck(self.hip.hipModuleLaunchKernel(self.function(name), grid, 1, 1, block, 1, 1, 0, None, params, None),
                 f"hipModuleLaunchKernel({name})")

    # ---- the operations of include/cera_hip_kernels.h -------------------------------------------
    def quantize_q8_0(self, x: np.ndarray):
        x = np.ascontiguousarray(x, np.float32)
        k = x.size
        assert k and k % 32 == 0
        dx, ds, dq = self.upload(x), self.malloc(k // 32 * 4), self.malloc(k)
        self.launch("cera_k_quantize_q8_0", (k // 4 + 255) // 256, 256, QuantizeArgs(dx, k, ds, dq, None))
        return self.download(ds, (k // 32,), np.float32), self.download(dq, (k,), np.int8), (ds, dq)

    def rmsnorm_q8_0(self, x: np.ndarray, w: np.ndarray, eps: float):
        n = x.size
        assert n % 32 == 0 and n <= 16384
        dx, dw = self.upload(np.asarray(x, np.float32)), self.upload(np.asarray(w, np.float32))
        dy, ds, dq = self.malloc(n * 4), self.malloc(n // 32 * 4), self.malloc(n)
        self.launch("cera_k_rmsnorm_q8_0", 1, 1024, RmsnormQ8Args(dx, dw, n, eps, dy, ds, dq))
        return self.download(dy, (n,), np.float32), self.download(ds, (n // 32,), np.float32), self.download(dq, (n,), np.int8)

    def gemv(self, ggml_type: int, blocks: np.ndarray, m: int, k: int, x: np.ndarray, resid: np.ndarray | None = None,
             n_cu: int = 256):
        """y = W . Q8_0(x) (+ resid): the quantizer, then the GEMV instance the header's rule selects."""
        elems, nbytes = BLOCK[ggml_type]
        unit = 64 if ggml_type in (12, 14) else 32
        n_units = k // unit
        ks = next(w for w in (1, 2, 4, 8) if n_units <= 64 * w)
        _, _, (ds, dq) = self.quantize_q8_0(x)
        dw = self.upload(np.ascontiguousarray(blocks).reshape(-1).view(np.uint8))
        dy = self.malloc(m * 4)
        dr = self.upload(np.asarray(resid, np.float32)) if resid is not None else None
        target = max(1, n_cu * 24 // ks)
        rows = (m + target - 1) // target
        rows = (rows + 1) // 2 * 2
        a = GemvArgs(dw, None, dq, ds, dy, dr, m, n_units, k // elems * nbytes, rows, None, 0, None)
        name = f"cera_k_gemv_{GGML_NAMES[ggml_type]}_ks{ks}_{'add' if resid is not None else 'store'}"
        self.launch(name, (m + rows - 1) // rows, 64 * ks, a)
        return self.download(dy, (m,), np.float32)
