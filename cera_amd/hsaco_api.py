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


# ---- the rest of a forward pass: argument structs of include/cera_hip_kernels.h ------------------
class EmbedTokenArgs(C.Structure):
    _fields_ = [("w", C.c_void_p), ("row_bytes", C.c_uint64), ("ggml_type", C.c_uint32), ("token", C.c_uint32),
                ("pos", C.c_uint32), ("k", C.c_uint32), ("scalars", C.c_void_p), ("scale", C.c_float), ("out", C.c_void_p)]


class EmbedRowsArgs(C.Structure):
    _fields_ = [("w", C.c_void_p), ("row_bytes", C.c_uint64), ("tokens", C.c_void_p), ("ggml_type", C.c_uint32),
                ("k", C.c_uint32), ("scale", C.c_float), ("out", C.c_void_p)]


class RmsnormRowsArgs(C.Structure):
    _fields_ = [("x", C.c_void_p), ("w", C.c_void_p), ("n", C.c_uint32), ("eps", C.c_float), ("y", C.c_void_p),
                ("scales", C.c_void_p), ("quants", C.c_void_p), ("bsum", C.c_void_p)]


class RopeKvArgs(C.Structure):
    _fields_ = [("q", C.c_void_p), ("k", C.c_void_p), ("v", C.c_void_p), ("cs_table", C.c_void_p), ("pos", C.c_void_p),
                ("n_heads", C.c_uint32), ("n_kv_heads", C.c_uint32), ("head_dim", C.c_uint32), ("rope_type", C.c_uint32),
                ("k_cache", C.c_void_p), ("v_cache", C.c_void_p), ("max_seq", C.c_uint32)]


class AttnDecodeArgs(C.Structure):
    _fields_ = [("q", C.c_void_p), ("kc", C.c_void_p), ("vc", C.c_void_p), ("seq_len", C.c_uint32), ("max_seq", C.c_uint32),
                ("scale", C.c_float), ("chunks_per_part", C.c_uint32), ("n_parts", C.c_uint32), ("q_stride", C.c_uint32),
                ("g_total", C.c_uint32), ("n_kv", C.c_uint32), ("n_queries", C.c_uint32), ("part_acc", C.c_void_p),
                ("part_ml", C.c_void_p)]


class AttnMergeArgs(C.Structure):
    _fields_ = [("part_acc", C.c_void_p), ("part_ml", C.c_void_p), ("n_parts", C.c_uint32), ("g_total", C.c_uint32),
                ("n_heads", C.c_uint32), ("n_pairs", C.c_uint32), ("out", C.c_void_p), ("scales", C.c_void_p),
                ("quants", C.c_void_p), ("bsum", C.c_void_p)]


class AttnPrefillArgs(C.Structure):
    _fields_ = [("q", C.c_void_p), ("kc", C.c_void_p), ("vc", C.c_void_p), ("first_len", C.c_uint32), ("n_queries", C.c_uint32),
                ("max_seq", C.c_uint32), ("scale", C.c_float), ("part_keys", C.c_uint32), ("n_parts", C.c_uint32),
                ("q_stride", C.c_uint32), ("part_acc", C.c_void_p), ("part_ml", C.c_void_p)]


class SiluMulArgs(C.Structure):
    _fields_ = [("gate", C.c_void_p), ("up", C.c_void_p), ("n", C.c_uint64), ("out", C.c_void_p), ("scales", C.c_void_p),
                ("quants", C.c_void_p), ("bsum", C.c_void_p)]


class ArgmaxPartialArgs(C.Structure):
    _fields_ = [("x", C.c_void_p), ("n", C.c_uint32), ("pv", C.c_void_p), ("pi", C.c_void_p)]


class ArgmaxFinalArgs(C.Structure):
    _fields_ = [("pv", C.c_void_p), ("pi", C.c_void_p), ("np", C.c_uint32), ("out", C.c_void_p), ("out2", C.c_void_p)]


class KvShiftArgs(C.Structure):
    _fields_ = [("src", C.c_void_p), ("dst", C.c_void_p), ("src_row", C.c_uint32), ("dst_row", C.c_uint32), ("n_rows", C.c_uint32),
                ("src_head_stride", C.c_uint64), ("dst_head_stride", C.c_uint64), ("delta_cs", C.c_void_p), ("rope_type", C.c_uint32)]


class GemmArgs(C.Structure):       # cera_k_gemm_args
    _fields_ = [("w", C.c_void_p), ("bq", C.c_void_p), ("bs", C.c_void_p), ("bsum", C.c_void_p), ("bh", C.c_void_p),
                ("out", C.c_void_p), ("m", C.c_uint32), ("n", C.c_uint32), ("k", C.c_uint32), ("row_bytes", C.c_uint32),
                ("ld_m", C.c_uint64), ("ld_n", C.c_uint64), ("resid", C.c_void_p), ("resid_scale", C.c_float),
                ("k_chunk", C.c_uint32), ("part_stride", C.c_uint64), ("w2", C.c_void_p), ("out2", C.c_void_p),
                ("m2", C.c_uint32), ("tiles1", C.c_uint32), ("ld_n2", C.c_uint64), ("hq", C.c_void_p), ("hs", C.c_void_p),
                ("hbsum", C.c_void_p), ("dbg_dots", C.c_void_p), ("bf8", C.c_void_p), ("hh", C.c_void_p)]


class GemmActFp8Args(C.Structure):
    _fields_ = [("quants", C.c_void_p), ("scales", C.c_void_p), ("bsum", C.c_void_p), ("out", C.c_void_p), ("n", C.c_uint32),
                ("k", C.c_uint32), ("halves", C.c_void_p)]


class GemmActF16Args(C.Structure):
    _fields_ = [("quants", C.c_void_p), ("out", C.c_void_p), ("n_words", C.c_uint64)]


def gemm_fp8_act_bytes(n: int, k: int) -> int:
    """CERA_K_GEMM_FP8_ACT_BYTES of the header."""
    return (n + 63) // 64 * 2 * (k // 256) * 21504


def rope_table(max_seq: int, head_dim: int, base: float, freq_factors=None) -> np.ndarray:
    """[max_seq][head_dim/2] (cos, sin) with the reference's recurrence (cera/src/backend/cpu.rs:5031-5045,
    5161-5180): theta_0 = pos as f32, theta_{i+1} = theta_i * base^(-2/head_dim) in f32, libm cosf / sinf."""
    libm = C.CDLL("libm.so.6")
    for f in (libm.cosf, libm.sinf, libm.powf):
        f.restype = C.c_float
    libm.cosf.argtypes = libm.sinf.argtypes = [C.c_float]
    libm.powf.argtypes = [C.c_float, C.c_float]
    half = head_dim // 2
    theta_scale = np.float32(libm.powf(C.c_float(base), C.c_float(-2.0 / head_dim)))
    out = np.empty((max_seq, half, 2), np.float32)
    for p in range(max_seq):
        theta = np.float32(p)
        for i in range(half):
            ang = np.float32(theta / np.float32(freq_factors[i])) if freq_factors is not None else theta
            out[p, i, 0] = libm.cosf(C.c_float(ang))
            out[p, i, 1] = libm.sinf(C.c_float(ang))
            theta = np.float32(theta * theta_scale)
    return out


def _launch3(host, name, grid, block, args):
    gx, gy, gz = (tuple(grid) + (1, 1))[:3] if isinstance(grid, (tuple, list)) else (grid, 1, 1)
    params = (C.c_void_p * 1)(C.cast(C.pointer(args), C.c_void_p))
    host._ck(host.hip.hipModuleLaunchKernel(host.function(name), gx, gy, gz, block, 1, 1, 0, None, params, None),
             f"hipModuleLaunchKernel({name})")


class Model:
    """LlamaModel::forward / ::forward_prefill (cera/src/model/llama.rs:468-597, 738-1523) for a dense llama
    with Q4_K / Q6_K / Q4_0 / Q4_1 / Q8_0 projection matrices, driven from the code object alone: every
    launch below is hipModuleLaunchKernel on a kernel of include/cera_hip_kernels.h, in the order and with
    the launch rules libcera_hip.so uses, so the logits carry the library's bits.  f32 KV cache, hidden and
    feed-forward widths up to 4096 (one pass per row), no biases / QK-norm / scalars other than 1.

    ``weights``: name -> (ggml_type, m, k, uint8 blocks) for matrices, name -> float32 array for norms."""

    def __init__(self, host: Host, cfg: dict, weights: dict, n_cu: int = 256):
        self.h, self.cfg, self.n_cu = host, dict(cfg), n_cu
        c = cfg
        self.hs, self.ffn, self.hd = c["hidden"], c["ffn"], c["head_dim"]
        self.nh, self.nkv, self.max_seq = c["n_heads"], c["n_kv_heads"], c["max_seq_len"]
        self.q_dim, self.kv_dim = self.nh * self.hd, self.nkv * self.hd
        self.eps, self.vocab = float(c.get("rms_eps", 1e-5)), c["vocab"]
        assert self.hd in (64, 128) and self.hs <= 4096 and self.ffn <= 4096 and (self.nh // self.nkv) in (1, 2, 4, 8)
        up = host.upload
        self.seq_len = 0

        def mat(name):
            t, m, k, blocks = weights[name]
            b = np.ascontiguousarray(blocks).reshape(-1).view(np.uint8)
            elems, nbytes = BLOCK[t]
            native = up(b)
            copy, crb = host.decode_copy(t, b, m, k)
            return dict(t=t, m=m, k=k, native=native, row_bytes=k // elems * nbytes, copy=copy, crb=crb)

        self.layers = []
        for i in range(c["n_layers"]):
            L = {n: mat(f"blk.{i}.{n}.weight") for n in ("attn_q", "attn_k", "attn_v", "attn_output", "ffn_gate", "ffn_up", "ffn_down")}
            # Q | K share one matrix, rows back to back (what the library's fused Q|K|V launch reads)
            tq, mq, k, bq = weights[f"blk.{i}.attn_q.weight"]
            tk, mk, _, bk = weights[f"blk.{i}.attn_k.weight"]
            assert tq == tk
            qk = np.concatenate([np.ascontiguousarray(bq).reshape(-1).view(np.uint8), np.ascontiguousarray(bk).reshape(-1).view(np.uint8)])
            copy, crb = host.decode_copy(tq, qk, mq + mk, k)
            L["qk"] = dict(t=tq, m=mq + mk, k=k, copy=copy, crb=crb)
            L["attn_norm"] = up(np.asarray(weights[f"blk.{i}.attn_norm.weight"], np.float32))
            L["ffn_norm"] = up(np.asarray(weights[f"blk.{i}.ffn_norm.weight"], np.float32))
            kv_bytes = self.nkv * self.max_seq * self.hd * 4
            L["kc"], L["vc"] = up(np.zeros(kv_bytes, np.uint8)), up(np.zeros(kv_bytes, np.uint8))
            self.layers.append(L)
        t, m, k, blocks = weights["token_embd.weight"]
        elems, nbytes = BLOCK.get(t, (1, 4))
        self.embd = dict(t=t, dev=up(np.ascontiguousarray(blocks).reshape(-1).view(np.uint8)), row_bytes=k // elems * nbytes)
        self.head = mat("output.weight") if "output.weight" in weights else mat("token_embd.weight")
        self.out_norm = up(np.asarray(weights["output_norm.weight"], np.float32))
        self.rope = up(rope_table(self.max_seq, self.hd, float(c.get("rope_theta", 10000.0))))
        self.rope_type = int(c.get("rope_type", 1))
        m4 = host.malloc
        self.scalars = m4(16)
        self.hidden, self.q = m4(self.hs * 4), m4((self.q_dim + 2 * self.kv_dim) * 4)
        self.k_, self.v_ = self.q + self.q_dim * 4, self.q + (self.q_dim + self.kv_dim) * 4
        self.attn = m4(self.q_dim * 4)
        maxk = max(self.hs, self.ffn, self.q_dim)
        self.xq, self.xs = m4(maxk), m4(maxk // 32 * 4)
        self.logits = m4(self.vocab * 4)
        self.acc, self.ml = m4(self.nkv * 1024 * (self.nh // self.nkv) * self.hd * 4), m4(self.nkv * 1024 * (self.nh // self.nkv) * 8)
        self.am_v, self.am_i, self.am_out = m4(1024 * 4), m4(1024 * 4), m4(4)
        self.pf_cap = 0

    def L(self, name, grid, block, args):
        _launch3(self.h, name, grid, block, args)

    # ---- single matrices ----------------------------------------------------------------------
    def _row_gemv(self, w, xs, xq, y, resid=None):
        name, p = GGML_NAMES[w["t"]], passes(w["t"], w["k"])
        kq = w["t"] in (12, 14)
        if p <= (1 if kq else 2):
            a = RowGemvArgs(w=w["copy"], m=w["m"], k=w["k"], row_bytes=w["crb"], rows_per_wave=2, xq=xq, xs=xs, y=y, resid=resid)
            self.L(f"cera_k_row_gemv_{name}_p{p}_{'add' if resid else 'store'}", (w["m"] + 7) // 8, 256, a)
        else:
            assert resid
            p = p if kq else (4 if p <= 4 else 8)
            a = RowGemvArgs(w=w["copy"], m=w["m"], k=w["k"], row_bytes=w["crb"], rows_per_wave=1, xq=xq, xs=xs, y=y, resid=resid)
            self.L(f"cera_k_row_gemv_long_{name}_p{p}_add", (w["m"] + 3) // 4, 256, a)

    def _attn_rule(self, last_len):
        """(g, S, chunks_per_part, n_parts) as the library picks them for one query and an f32 cache."""
        G = self.nh // self.nkv
        g = G // 2 if (G == 8 or (G == 4 and last_len < 16384)) else G
        split = g != G
        if split:
            S = 4 if last_len >= 1024 else 1
        else:
            S = 8 if last_len >= 8192 else (4 if last_len >= 2048 else (2 if last_len >= 1024 else 1))
        assert S in (1, 4), "this host carries the S = 1 and S = 4 instances"
        n_chunks = (last_len + 8 * S - 1) // (8 * S)
        want = max(1, min(1024, self.n_cu * 4 // self.nkv))
        cpp = max(1, (n_chunks + want - 1) // want)
        best, first, subs = None, cpp, G // g
        c = first
        while c <= n_chunks:
            parts = (n_chunks + c - 1) // c
            if c > first and parts * 4 < want:
                break
            groups = (parts + 3) // 4 * self.nkv * subs
            rnd = self.n_cu * (2 if G == 8 else 1)
            cost = c * ((groups + rnd - 1) // rnd)
            if best is None or cost < best:
                best, cpp = cost, c
            c += 1
        return g, S, cpp, (n_chunks + cpp - 1) // cpp

    # ---- LlamaModel::forward -------------------------------------------------------------------
    def forward(self, token: int, pos: int) -> np.ndarray:
        assert pos == self.seq_len and pos < self.max_seq
        e = self.embd
        self.L("cera_k_embed_token", (self.hs + 255) // 256, 256,
               EmbedTokenArgs(e["dev"], e["row_bytes"], e["t"], token, pos, self.hs, self.scalars, 1.0, self.hidden))
        scale = 1.0 / float(np.sqrt(np.float32(self.hd)))
        G = self.nh // self.nkv
        for Ly in self.layers:
            qk, v = Ly["qk"], Ly["attn_v"]
            R = 2 if (qk["m"] + v["m"]) >= 8 * self.n_cu else 1
            per = 8 * R
            p = RowGemvPairArgs()
            p.a = RowGemvArgs(w=qk["copy"], m=qk["m"], k=qk["k"], row_bytes=qk["crb"], rows_per_wave=R, x=self.hidden,
                              norm_w=Ly["attn_norm"], eps=self.eps, y=self.q)
            p.b = RowGemvArgs(w=v["copy"], m=v["m"], k=v["k"], row_bytes=v["crb"], rows_per_wave=R, x=self.hidden,
                              norm_w=Ly["attn_norm"], eps=self.eps, y=self.v_)
            p.n_blocks_a = (qk["m"] + per - 1) // per
            self.L(f"cera_k_norm_qkv_{GGML_NAMES[qk['t']]}_{GGML_NAMES[v['t']]}_p{passes(qk['t'], qk['k'])}_r{R}",
                   p.n_blocks_a + (v["m"] + per - 1) // per, 512, p)
            self.L("cera_k_rope_kv_f32", (self.nh + 2 * self.nkv, 1), self.hd // 2,
                   RopeKvArgs(self.q, self.k_, self.v_, self.rope, self.scalars + 4, self.nh, self.nkv, self.hd, self.rope_type,
                              Ly["kc"], Ly["vc"], self.max_seq))
            g, S, cpp, n_parts = self._attn_rule(pos + 1)
            groups = (n_parts + 3) // 4 * self.nkv
            self.L(f"cera_k_attn_decode_partial_f32_hd{self.hd}_g{g}_s{S}", (groups + 7) // 8 * 8 * (G // g), 256,
                   AttnDecodeArgs(self.q, Ly["kc"], Ly["vc"], pos + 1, self.max_seq, scale, cpp, n_parts, self.q_dim, G, self.nkv, 1,
                                  self.acc, self.ml))
            self.L(f"cera_k_attn_decode_merge_hd{self.hd}_q8_0", (self.nh, 1), 256,
                   AttnMergeArgs(self.acc, self.ml, n_parts, G, self.nh, 0, self.attn, self.xs, self.xq, None))
            self._row_gemv(Ly["attn_output"], self.xs, self.xq, self.hidden, self.hidden)
            gt, ut = Ly["ffn_gate"], Ly["ffn_up"]
            a = RowGemvArgs(w=gt["copy"], w2=ut["copy"], m=gt["m"], k=gt["k"], row_bytes=gt["crb"], rows_per_wave=4, x=self.hidden,
                            norm_w=Ly["ffn_norm"], eps=self.eps, out_q=self.xq, out_s=self.xs)
            self.L(f"cera_k_norm_gate_up_{GGML_NAMES[gt['t']]}_p{passes(gt['t'], gt['k'])}", (gt["m"] + 63) // 64, 1024, a)
            self._row_gemv(Ly["ffn_down"], self.xs, self.xq, self.hidden, self.hidden)
        self.L("cera_k_rmsnorm_q8_0", 1, 1024, RmsnormQ8Args(self.hidden, self.out_norm, self.hs, self.eps, self.hidden, self.xs, self.xq))
        self._row_gemv(self.head, self.xs, self.xq, self.logits)
        self.seq_len = pos + 1
        return self.h.download(self.logits, (self.vocab,), np.float32)

    def argmax(self) -> int:
        """The token of the logits the last call left on the device (two launches, four bytes back)."""
        np_ = max(1, min(1024, (self.vocab + 1023) // 1024))
        self.L("cera_k_argmax_partial", np_, 256, ArgmaxPartialArgs(self.logits, self.vocab, self.am_v, self.am_i))
        self.L("cera_k_argmax_final", 1, 256, ArgmaxFinalArgs(self.am_v, self.am_i, np_, self.am_out, None))
        return int(self.h.download(self.am_out, (1,), np.uint32)[0])

    # ---- LlamaModel::forward_prefill (batched route) ---------------------------------------------
    def _pf_buffers(self, n):
        if self.pf_cap >= n:
            return
        m4, maxk = self.h.malloc, max(self.hs, self.ffn, self.q_dim)
        self.pf = dict(hidden=m4(n * self.hs * 4), normed=m4(n * self.hs * 4), q=m4(n * self.q_dim * 4), k=m4(n * self.kv_dim * 4),
                       v=m4(n * self.kv_dim * 4), attn=m4(n * self.q_dim * 4), gate=m4(n * self.ffn * 4), up=m4(n * self.ffn * 4),
                       xq=m4(n * maxk), xh=m4(n * maxk * 2), x8=m4(gemm_fp8_act_bytes(n, maxk)), xs=m4(n * (maxk // 32) * 4),
                       bsum=m4(n * (maxk // 32) * 4), tokens=m4(n * 4),
                       acc=m4(n * self.nh * 8 * self.hd * 4), ml=m4(n * self.nh * 8 * 8))
        self.pf_cap = n

    def _gemm(self, w, n, out, resid=None, staged=None):
        """out[n][m] = B . W^T (+ resid) on the activations in pf xq / xs / bsum; `staged` remembers which
        re-laid copies (f16, fp8) of those activations are current."""
        P, t, m, k = self.pf, w["t"], w["m"], w["k"]
        a = GemmArgs(w=w["native"], bq=P["xq"], bs=P["xs"], bsum=P["bsum"], out=out, m=m, n=n, k=k, row_bytes=w["row_bytes"],
                     ld_m=1, ld_n=m, resid=resid, resid_scale=1.0, k_chunk=k, part_stride=0, m2=0, tiles1=(m + 127) // 128, ld_n2=0)
        if t == 14:
            if not staged.get("f16"):
                words = n * k // 16
                self.L("cera_k_gemm_act_f16", (words + 255) // 256, 256, GemmActF16Args(P["xq"], P["xh"], words))
                staged["f16"] = True
            a.bh = P["xh"]
        if t == 12:
            if not staged.get("fp8"):
                self.L("cera_k_gemm_act_fp8", (n + 63) // 64 * 2 * (k // 256), 256, GemmActFp8Args(P["xq"], P["xs"], P["bsum"], P["x8"], n, k))
                staged["fp8"] = True
            a.bf8 = P["x8"]
        self.L(f"cera_k_gemm_{GGML_NAMES[t]}", ((n + 63) // 64, (m + 127) // 128, 1), 256, a)

    def forward_prefill(self, tokens, start_pos: int) -> np.ndarray:
        """16 tokens or more at once (at most 1024 keys in all, hidden and ffn below 2048 so the tile GEMMs need no K split): logits of the last."""
        n = len(tokens)
        assert n >= 16 and start_pos == self.seq_len and start_pos + n <= min(self.max_seq, 1024) and max(self.hs, self.ffn) < 2048
        self._pf_buffers(n)
        P, e, G = self.pf, self.embd, self.nh // self.nkv
        self.h._ck(self.h.hip.hipMemcpy(C.c_void_p(P["tokens"]), C.c_void_p(np.ascontiguousarray(tokens, np.uint32).ctypes.data),
                                        C.c_size_t(4 * n), 1), "hipMemcpy tokens")
        self.h._ck(self.h.hip.hipMemcpy(C.c_void_p(self.scalars + 4), C.c_void_p(np.array([start_pos], np.uint32).ctypes.data),
                                        C.c_size_t(4), 1), "hipMemcpy pos")
        self.L("cera_k_embed_rows", ((self.hs + 255) // 256, n), 256, EmbedRowsArgs(e["dev"], e["row_bytes"], P["tokens"], e["t"], self.hs, 1.0, P["hidden"]))
        scale = 1.0 / float(np.sqrt(np.float32(self.hd)))
        last_len = start_pos + n
        part_keys = 128
        n_parts = (last_len + part_keys - 1) // part_keys
        for Ly in self.layers:
            st = {}
            self.L("cera_k_rmsnorm_rows_q8_0", n, 256, RmsnormRowsArgs(P["hidden"], Ly["attn_norm"], self.hs, self.eps, P["normed"], P["xs"], P["xq"], P["bsum"]))
            self._gemm(Ly["attn_q"], n, P["q"], staged=st)
            self._gemm(Ly["attn_k"], n, P["k"], staged=st)
            self._gemm(Ly["attn_v"], n, P["v"], staged=st)
            self.L("cera_k_rope_kv_f32", (self.nh + 2 * self.nkv, n), self.hd // 2,
                   RopeKvArgs(P["q"], P["k"], P["v"], self.rope, self.scalars + 4, self.nh, self.nkv, self.hd, self.rope_type,
                              Ly["kc"], Ly["vc"], self.max_seq))
            if n >= 16:
                self.L(f"cera_k_attn_prefill_partial_f32_hd{self.hd}_g{G}", ((n + 31) // 32, self.nkv, n_parts), 64 * G,
                       AttnPrefillArgs(P["q"], Ly["kc"], Ly["vc"], start_pos + 1, n, self.max_seq, scale, part_keys, n_parts, self.q_dim, P["acc"], P["ml"]))
                self.L(f"cera_k_attn_prefill_merge_hd{self.hd}_q8_0", (self.nh * n + 7) // 8, 256,
                       AttnMergeArgs(P["acc"], P["ml"], n_parts, G, self.nh, self.nh * n, P["attn"], P["xs"], P["xq"], P["bsum"]))
            else:
                raise NotImplementedError("9-15 tokens: the decode kernels with n_queries, not wired in this host")
            st = {}
            self._gemm(Ly["attn_output"], n, P["hidden"], resid=P["hidden"], staged=st)
            st = {}
            self.L("cera_k_rmsnorm_rows_q8_0", n, 256, RmsnormRowsArgs(P["hidden"], Ly["ffn_norm"], self.hs, self.eps, P["normed"], P["xs"], P["xq"], P["bsum"]))
            self._gemm(Ly["ffn_gate"], n, P["gate"], staged=st)
            self._gemm(Ly["ffn_up"], n, P["up"], staged=st)
            tot = n * self.ffn
            self.L("cera_k_silu_mul_q8_0", (tot // 4 + 255) // 256, 256, SiluMulArgs(P["gate"], P["up"], tot, P["gate"], P["xs"], P["xq"], P["bsum"]))
            st = {}
            self._gemm(Ly["ffn_down"], n, P["hidden"], resid=P["hidden"], staged=st)
        self.seq_len = start_pos + n
        last = P["hidden"] + (n - 1) * self.hs * 4
        self.L("cera_k_rmsnorm_rows_q8_0", 1, 256, RmsnormRowsArgs(last, self.out_norm, self.hs, self.eps, self.hidden, self.xs, self.xq, None))
        self._row_gemv(self.head, self.xs, self.xq, self.logits)
        return self.h.download(self.logits, (self.vocab,), np.float32)
