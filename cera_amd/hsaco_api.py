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


class DecodeCopyArgs(C.Structure):  # cera_k_decode_copy_args
    _fields_ = [("src", C.c_void_p), ("dst", C.c_void_p), ("n_units", C.c_uint32), ("row_bytes", C.c_uint32),
                ("copy_row_bytes", C.c_uint32)]


class RowGemvArgs(C.Structure):    # cera_k_row_gemv_args
    _fields_ = [("w", C.c_void_p), ("w2", C.c_void_p), ("m", C.c_uint32), ("k", C.c_uint32), ("row_bytes", C.c_uint32),
                ("rows_per_wave", C.c_uint32), ("xq", C.c_void_p), ("xs", C.c_void_p), ("x", C.c_void_p),
                ("norm_w", C.c_void_p), ("eps", C.c_float), ("y", C.c_void_p), ("resid", C.c_void_p),
                ("out_q", C.c_void_p), ("out_s", C.c_void_p)]


class RowGemvPairArgs(C.Structure):  # cera_k_row_gemv_pair_args
    _fields_ = [("a", RowGemvArgs), ("b", RowGemvArgs), ("n_blocks_a", C.c_uint32)]


def _up128(b: int) -> int:
    return (b + 127) & ~127


def decode_copy_row_bytes(ggml_type: int, k: int) -> int:
    """CERA_K_DECODE_COPY_ROW_BYTES of the header."""
    if ggml_type == 12:
        return _up128(4 * (k // 64)) + 2 * _up128(16 * (k // 64))
    if ggml_type == 14:
        return 3 * _up128(16 * (k // 64)) + _up128(4 * (k // 64)) + _up128(k // 128)
    if ggml_type == 2:
        return _up128(2 * (k // 32)) + _up128(16 * (k // 32))
    if ggml_type == 3:
        return _up128(4 * (k // 32)) + _up128(16 * (k // 32))
    return _up128(2 * (k // 32)) + 2 * _up128(16 * (k // 32))


def passes(ggml_type: int, k: int) -> int:
    unit = 64 if ggml_type in (12, 14) else 32
    return (k // unit + 63) // 64


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

    # ---- the one-wavefront-per-row kernels on decode copies --------------------------------------
    def decode_copy(self, ggml_type: int, blocks: np.ndarray, m: int, k: int):
        """Uploads native rows and builds their decode copy: (device pointer, row stride)."""
        elems, nbytes = BLOCK[ggml_type]
        unit = 64 if ggml_type in (12, 14) else 32
        assert k % elems == 0 and k <= 16384
        src = self.upload(np.ascontiguousarray(blocks).reshape(-1).view(np.uint8))
        crb = decode_copy_row_bytes(ggml_type, k)
        dst = self.malloc(crb * m)
        self.launch(f"cera_k_decode_copy_{GGML_NAMES[ggml_type]}", m, 256,
                    DecodeCopyArgs(src, dst, k // unit, k // elems * nbytes, crb))
        return dst, crb

    def row_gemv(self, ggml_type: int, blocks: np.ndarray, m: int, k: int, x: np.ndarray, resid: np.ndarray | None = None):
        """y = W . Q8_0(x) (+ resid) from the decode copy: the short-row kernel up to k = 4096, the
        long-row kernel (residual form only) beyond."""
        name = GGML_NAMES[ggml_type]
        p = passes(ggml_type, k)
        dw, crb = self.decode_copy(ggml_type, blocks, m, k)
        _, _, (ds, dq) = self.quantize_q8_0(x)
        dy = self.malloc(m * 4)
        dr = self.upload(np.asarray(resid, np.float32)) if resid is not None else None
        kq = ggml_type in (12, 14)
        if k <= 4096 and p <= (1 if kq else 2):
            a = RowGemvArgs(w=dw, m=m, k=k, row_bytes=crb, rows_per_wave=2, xq=dq, xs=ds, y=dy, resid=dr)
            self.launch(f"cera_k_row_gemv_{name}_p{p}_{'add' if resid is not None else 'store'}", (m + 7) // 8, 256, a)
        else:
            assert resid is not None, "the long-row kernel exists in the residual form"
            p = p if kq else (4 if p <= 4 else 8)
            a = RowGemvArgs(w=dw, m=m, k=k, row_bytes=crb, rows_per_wave=1, xq=dq, xs=ds, y=dy, resid=dr)
            self.launch(f"cera_k_row_gemv_long_{name}_p{p}_add", (m + 3) // 4, 256, a)
        return self.download(dy, (m,), np.float32)

    def norm_gate_up(self, ggml_type: int, gate: np.ndarray, up: np.ndarray, m: int, k: int, x, norm_w, eps: float):
        """Q8_0(silu(gate.n) * (up.n)), n = Q8_0(rmsnorm(x, norm_w)): (quants [m], scales [m/32])."""
        assert m % 32 == 0 and k <= 4096
        dg, crb = self.decode_copy(ggml_type, gate, m, k)
        du, _ = self.decode_copy(ggml_type, up, m, k)
        dx, dn = self.upload(np.asarray(x, np.float32)), self.upload(np.asarray(norm_w, np.float32))
        dq, ds = self.malloc(m), self.malloc(m // 32 * 4)
        a = RowGemvArgs(w=dg, w2=du, m=m, k=k, row_bytes=crb, rows_per_wave=4, x=dx, norm_w=dn, eps=eps, out_q=dq, out_s=ds)
        self.launch(f"cera_k_norm_gate_up_{GGML_NAMES[ggml_type]}_p{passes(ggml_type, k)}", (m + 63) // 64, 1024, a)
        return self.download(dq, (m,), np.int8), self.download(ds, (m // 32,), np.float32)

    def norm_qkv(self, type_a: int, wa: np.ndarray, ma: int, type_b: int, wb: np.ndarray, mb: int, k: int, x, norm_w,
                 eps: float, rows_per_wave: int = 2):
        """(A . n, B . n), n = Q8_0(rmsnorm(x, norm_w)), in one launch."""
        assert k <= 4096 and rows_per_wave in (1, 2)
        da, crb_a = self.decode_copy(type_a, wa, ma, k)
        db, crb_b = self.decode_copy(type_b, wb, mb, k)
        dx, dn = self.upload(np.asarray(x, np.float32)), self.upload(np.asarray(norm_w, np.float32))
        dya, dyb = self.malloc(ma * 4), self.malloc(mb * 4)
        per = 8 * rows_per_wave
        p = RowGemvPairArgs()
        p.a = RowGemvArgs(w=da, m=ma, k=k, row_bytes=crb_a, rows_per_wave=rows_per_wave, x=dx, norm_w=dn, eps=eps, y=dya)
        p.b = RowGemvArgs(w=db, m=mb, k=k, row_bytes=crb_b, rows_per_wave=rows_per_wave, x=dx, norm_w=dn, eps=eps, y=dyb)
        p.n_blocks_a = (ma + per - 1) // per
        name = f"cera_k_norm_qkv_{GGML_NAMES[type_a]}_{GGML_NAMES[type_b]}_p{passes(type_a, k)}_r{rows_per_wave}"
        self.launch(name, p.n_blocks_a + (mb + per - 1) // per, 512, p)
        return self.download(dya, (ma,), np.float32), self.download(dyb, (mb,), np.float32)
