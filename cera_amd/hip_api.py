"""ctypes binding of the C-ABI HIP library (``include/cera_hip.h``).

This is plumbing for the tests and the benchmark: every call goes straight to
``libcera_hip.so``.  There is no CPU fallback -- if the library or a GPU is
missing, loading fails with an error.
"""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import _build

F32, F16, Q4_0, Q4_1, Q8_0, Q4_K, Q5_K, Q6_K, BF16 = 0, 1, 2, 3, 8, 12, 13, 14, 30
STATUS = {0: "OK", 1: "ERR_DEVICE", 2: "ERR_OOM", 3: "ERR_UNSUPPORTED_DTYPE", 4: "ERR_SHAPE", 5: "ERR_POSITION",
          6: "ERR_ARGUMENT"}

# every symbol include/cera_hip.h declares
SYMBOLS = [
    "cera_hip_ctx_create", "cera_hip_ctx_destroy", "cera_hip_ctx_set_decode_copies", "cera_hip_decode_copy_reserve_bytes", "cera_hip_decode_copy_plan", "cera_hip_drop_decode_copies", "cera_hip_last_error", "cera_hip_sync", "cera_hip_device_info",
    "cera_hip_malloc", "cera_hip_free", "cera_hip_upload", "cera_hip_download", "cera_hip_copy_dev", "cera_hip_copy_kernel",
    "cera_hip_event_create", "cera_hip_event_destroy", "cera_hip_event_record", "cera_hip_event_elapsed_ms",
    "cera_hip_tensor_upload", "cera_hip_tensor_clone", "cera_hip_tensor_free", "cera_hip_tensor_nbytes",
    "cera_hip_quantize_q8_0", "cera_hip_gemv", "cera_hip_gemm", "cera_hip_attn_decode", "cera_hip_attn_prefill", "cera_hip_rmsnorm",
    "cera_hip_silu_mul", "cera_hip_rope", "cera_hip_argmax", "cera_hip_dequantize_row",
    "cera_hip_quantize_q8_0_dev", "cera_hip_gemv_q8_dev", "cera_hip_gemv_seq_dev", "cera_hip_decode_ops_dev", "cera_hip_attn_decode_dev",
    "cera_hip_gemm_dev",
    "cera_hip_model_create", "cera_hip_model_destroy", "cera_hip_forward", "cera_hip_forward_greedy",
    "cera_hip_forward_prefill", "cera_hip_forward_prefill_logits_all", "cera_hip_truncate_kv", "cera_hip_gemv_pair", "cera_hip_gemm_pair", "cera_hip_gemm_swiglu", "cera_hip_gemm_swiglu_f16", "cera_hip_gemv_nb", "cera_hip_configure_kv", "cera_hip_kv_type", "cera_hip_attn_f16kv",
    "cera_hip_attn_decode_f16_dev", "cera_hip_shift_kv", "cera_hip_write_kv", "cera_hip_set_seq_len", "cera_hip_seq_len", "cera_hip_memory_bytes",
    "cera_hip_read_kv", "cera_hip_read_hidden",
    "cera_hip_gemv_reference_order", "cera_hip_attn_decode_reference_order", "cera_hip_rmsnorm_reference_order",
    "cera_hip_gemm_reference_order", "cera_hip_flash_attn_reference_order",
    "cera_hip_set_reference_order", "cera_hip_reference_order",
    "cera_hip_rmsnorm_q8_0", "cera_hip_attn_decode_step", "cera_hip_attn_decode_dev_noalloc", "cera_hip_gemm_block_dots",
    "cera_hip_ffn_gate_up_fused", "cera_hip_qkv_fused",
]


class HipError(RuntimeError):
    def __init__(self, status: int, message: str):
        super().__init__(f"cera_hip {STATUS.get(status, status)}: {message}")
        self.status = status
        self.message = message


class Tensor(C.Structure):
    _fields_ = [("ggml_type", C.c_uint32), ("_reserved", C.c_uint32), ("m", C.c_uint64), ("k", C.c_uint64),
                ("data", C.c_void_p), ("nbytes", C.c_uint64)]


class Layer(C.Structure):
    _fields_ = [("attn_norm", C.c_void_p), ("ffn_norm", C.c_void_p),
                ("attn_q", Tensor), ("attn_k", Tensor), ("attn_v", Tensor), ("attn_output", Tensor),
                ("ffn_gate", Tensor), ("ffn_up", Tensor), ("ffn_down", Tensor),
                ("q_bias", C.c_void_p), ("k_bias", C.c_void_p), ("v_bias", C.c_void_p),
                ("q_norm", C.c_void_p), ("k_norm", C.c_void_p)]


class Config(C.Structure):
    _fields_ = [("n_layers", C.c_uint32), ("hidden", C.c_uint32), ("ffn", C.c_uint32), ("n_heads", C.c_uint32),
                ("n_kv_heads", C.c_uint32), ("head_dim", C.c_uint32), ("vocab", C.c_uint32),
                ("max_seq_len", C.c_uint32), ("rope_type", C.c_uint32),
                ("rope_theta", C.c_float), ("rms_eps", C.c_float), ("embed_scale", C.c_float),
                ("residual_scale", C.c_float), ("attn_scale", C.c_float), ("logit_scale", C.c_float),
                ("rope_freqs", C.c_void_p)]


class GemvOp(C.Structure):
    _fields_ = [("w", C.c_void_p), ("w2", C.c_void_p), ("xs", C.c_void_p), ("xq", C.c_void_p), ("y", C.c_void_p)]


class DecodeOp(C.Structure):
    """cera_hip_decode_op (include/cera_hip.h)."""
    GEMV, NORM_GEMV, NORM_GATE_UP, NORM_QUANT, QUANT = range(5)
    _fields_ = [("kind", C.c_uint32), ("n", C.c_uint32), ("w", C.c_void_p), ("w2", C.c_void_p), ("x", C.c_void_p),
                ("norm_w", C.c_void_p), ("eps", C.c_float), ("xs", C.c_void_p), ("xq", C.c_void_p), ("resid", C.c_void_p),
                ("y", C.c_void_p), ("y2", C.c_void_p), ("out_s", C.c_void_p), ("out_q", C.c_void_p)]


_lib = None


def load_library() -> C.CDLL:
    """Load libcera_hip.so (never builds it: build with ``__graft_entry__.build()``)."""
    global _lib
    if _lib is not None:
        return _lib
    if not _build.HIP_LIB.exists():
        raise RuntimeError(f"{_build.HIP_LIB} is missing: run `python -c 'import __graft_entry__ as g; g.build()'`")
    L = C.CDLL(str(_build.HIP_LIB))
    vp, u32, u64, f32, i32 = C.c_void_p, C.c_uint32, C.c_uint64, C.c_float, C.c_int
    pp = C.POINTER(C.c_void_p)
    sig = {
        "cera_hip_ctx_create": (i32, [i32, C.c_char_p, pp]), "cera_hip_ctx_destroy": (None, [vp]),
        "cera_hip_ctx_set_decode_copies": (i32, [vp, i32]),
        "cera_hip_decode_copy_reserve_bytes": (u64, [vp]),
        "cera_hip_decode_copy_plan": (u64, [vp, u32, u64, u64, vp]),
        "cera_hip_drop_decode_copies": (i32, [vp, vp]),
        "cera_hip_last_error": (C.c_char_p, [vp]), "cera_hip_sync": (i32, [vp]),
        "cera_hip_device_info": (i32, [vp, C.c_char_p, C.POINTER(u32), C.POINTER(u64)]),
        "cera_hip_malloc": (i32, [vp, u64, pp]), "cera_hip_free": (i32, [vp, vp]),
        "cera_hip_upload": (i32, [vp, vp, vp, u64]), "cera_hip_download": (i32, [vp, vp, vp, u64]),
        "cera_hip_copy_dev": (i32, [vp, vp, vp, u64]),
        "cera_hip_copy_kernel": (i32, [vp, vp, vp, u64]),
        "cera_hip_event_create": (i32, [vp, pp]), "cera_hip_event_destroy": (None, [vp]),
        "cera_hip_event_record": (i32, [vp, vp]),
        "cera_hip_event_elapsed_ms": (i32, [vp, vp, vp, C.POINTER(f32)]),
        "cera_hip_tensor_upload": (i32, [vp, C.POINTER(Tensor), pp]),
        "cera_hip_tensor_clone": (i32, [vp, vp, pp]),
        "cera_hip_tensor_free": (None, [vp, vp]), "cera_hip_tensor_nbytes": (u64, [vp]),
        "cera_hip_quantize_q8_0": (i32, [vp, vp, u64, vp, vp]),
        "cera_hip_gemv": (i32, [vp, C.POINTER(Tensor), vp, vp, vp, vp]),
        "cera_hip_gemm": (i32, [vp, C.POINTER(Tensor), vp, u64, vp]),
        "cera_hip_attn_decode": (i32, [vp, vp, vp, vp, u32, u32, u32, u64, f32, u32, vp]),
        "cera_hip_attn_prefill": (i32, [vp, vp, vp, vp, u32, u32, u32, u64, u32, f32, vp]),
        "cera_hip_rmsnorm": (i32, [vp, vp, vp, u64, f32, vp]),
        "cera_hip_silu_mul": (i32, [vp, vp, vp, u64, vp]),
        "cera_hip_rope": (i32, [vp, vp, vp, u32, u32, u32, u32, f32, u32, vp]),
        "cera_hip_argmax": (i32, [vp, vp, u64, C.POINTER(u32)]),
        "cera_hip_dequantize_row": (i32, [vp, C.POINTER(Tensor), u64, vp]),
        "cera_hip_quantize_q8_0_dev": (i32, [vp, vp, u64, vp, vp]),
        "cera_hip_gemv_q8_dev": (i32, [vp, vp, vp, vp, vp]),
        "cera_hip_gemv_seq_dev": (i32, [vp, C.POINTER(GemvOp), u32]),
        "cera_hip_decode_ops_dev": (i32, [vp, C.POINTER(DecodeOp), u32]),
        "cera_hip_attn_decode_dev": (i32, [vp, vp, vp, vp, u32, u32, u32, u64, u64, f32, u32, vp]),
        "cera_hip_gemm_dev": (i32, [vp, vp, vp, u64, vp]),
        "cera_hip_model_create": (i32, [vp, C.POINTER(Config), C.POINTER(Tensor), C.POINTER(Tensor), vp,
                                        C.POINTER(Layer), pp]),
        "cera_hip_model_destroy": (None, [vp]),
        "cera_hip_forward": (i32, [vp, u32, u32, vp]),
        "cera_hip_forward_greedy": (i32, [vp, u32, u32, C.POINTER(u32)]),
        "cera_hip_forward_prefill": (i32, [vp, vp, u32, u32, vp]),
        "cera_hip_forward_prefill_logits_all": (i32, [vp, vp, u32, u32, vp]),
        "cera_hip_truncate_kv": (i32, [vp, u32]),
        "cera_hip_gemv_pair": (i32, [vp, vp, vp, vp, vp, vp]),
        "cera_hip_gemm_pair": (i32, [vp, vp, vp, vp, u64, vp, vp]),
        "cera_hip_gemm_swiglu": (i32, [vp, vp, vp, vp, u64, vp, vp, vp]),
        "cera_hip_gemm_swiglu_f16": (i32, [vp, vp, vp, vp, u64, vp, vp, vp, vp]),
        "cera_hip_gemv_nb": (i32, [vp, vp, vp, u32, vp]),
        "cera_hip_configure_kv": (i32, [vp, u32]),
        "cera_hip_kv_type": (u32, [vp]),
        "cera_hip_attn_f16kv": (i32, [vp, vp, vp, vp, u32, u32, u32, u64, u32, f32, u32, vp]),
        "cera_hip_attn_decode_f16_dev": (i32, [vp, vp, vp, vp, u32, u32, u32, u64, u64, f32, u32, vp]),
        "cera_hip_shift_kv": (i32, [vp, u32, u32]),
        "cera_hip_write_kv": (i32, [vp, u32, vp, vp, u32]),
        "cera_hip_set_seq_len": (i32, [vp, u32]),
        "cera_hip_seq_len": (u32, [vp]), "cera_hip_memory_bytes": (u64, [vp]),
        "cera_hip_read_kv": (i32, [vp, u32, vp, vp]), "cera_hip_read_hidden": (i32, [vp, vp]),
        "cera_hip_gemv_reference_order": (i32, [vp, C.POINTER(Tensor), vp, vp]),
        "cera_hip_attn_decode_reference_order": (i32, [vp, vp, vp, vp, u32, u32, u32, u64, f32, vp]),
        "cera_hip_rmsnorm_reference_order": (i32, [vp, vp, vp, u64, f32, vp]),
        "cera_hip_gemm_reference_order": (i32, [vp, C.POINTER(Tensor), vp, u64, u32, vp]),
        "cera_hip_flash_attn_reference_order": (i32, [vp, vp, vp, vp, u32, u32, u32, u32, u32, f32, vp]),
        "cera_hip_set_reference_order": (i32, [vp, u32]), "cera_hip_reference_order": (u32, [vp]),
        "cera_hip_attn_decode_dev_noalloc": (i32, [vp, vp, vp, vp, u32, u32, u32, u64, u64, f32, u32, vp]),
        "cera_hip_ffn_gate_up_fused": (i32, [vp, vp, vp, vp, vp, f32, vp, vp]),
        "cera_hip_qkv_fused": (i32, [vp, vp, vp, vp, vp, f32, vp, vp]),
        "cera_hip_gemm_block_dots": (i32, [vp, C.POINTER(Tensor), vp, u64, vp, vp]),
        "cera_hip_rmsnorm_q8_0": (i32, [vp, vp, vp, u64, f32, vp, vp, vp]),
        "cera_hip_attn_decode_step": (i32, [vp, vp, vp, vp, vp, vp, u32, u32, u32, u32, f32, u32, vp, f32, u32,
                                            vp, vp, vp, vp, vp]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(L, name)
        fn.restype, fn.argtypes = res, args
    _lib = L
    return L


def _p(a: np.ndarray) -> int:
    assert a.flags["C_CONTIGUOUS"]
    return a.ctypes.data


def make_config(cfg: dict) -> "Config":
    c = Config()
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
    return c


def decode_copy_reserve_bytes(cfg: dict) -> int:
    """Bytes model_create keeps free when it hands out decode copies (plain arithmetic, no GPU)."""
    c = make_config(cfg)
    return int(load_library().cera_hip_decode_copy_reserve_bytes(C.addressof(c)))


def decode_copy_plan(copy_bytes, free_bytes: int, reserve_bytes: int):
    """(taken mask, bytes taken) of model_create's decode-copy rule (plain arithmetic, no GPU)."""
    b = np.ascontiguousarray(copy_bytes, np.uint64)
    take = np.zeros(b.size, np.uint8)
    used = load_library().cera_hip_decode_copy_plan(_p(b), b.size, int(free_bytes), int(reserve_bytes), _p(take))
    return take.astype(bool), int(used)


def make_tensor(ggml_type: int, m: int, k: int, blocks: np.ndarray) -> Tensor:
    blocks = np.ascontiguousarray(blocks).reshape(-1).view(np.uint8)
    t = Tensor(ggml_type, 0, m, k, blocks.ctypes.data, blocks.size)
    t._keep = blocks  # keep the host bytes alive as long as the descriptor
    return t


class Context:
    """One HIP device + stream (cera_hip_ctx)."""

    def __init__(self, device: int = 0, hsaco_path: str | None = None):
        """hsaco_path: the standalone code object (``_build.HSACO``) to launch the quantizer and the
        GEMV instances from with hipModuleLaunchKernel; None = the kernels embedded in the library."""
        self.lib = load_library()
        h = C.c_void_p()
        st = self.lib.cera_hip_ctx_create(device, hsaco_path.encode() if hsaco_path else None, C.byref(h))
        if st != 0:
            raise HipError(st, (self.lib.cera_hip_last_error(None) or b"").decode())
        self.h = h

    # -- helpers
    def check(self, st: int):
        if st != 0:
            raise HipError(st, (self.lib.cera_hip_last_error(self.h) or b"").decode())

    def close(self):
        if getattr(self, "h", None):
            self.lib.cera_hip_ctx_destroy(self.h)
            self.h = None

    def sync(self):
        self.check(self.lib.cera_hip_sync(self.h))

    def set_decode_copies(self, enabled: bool):
        """Whether matrices prepared from now on get the permuted second copy the decode GEMVs stream."""
        self.check(self.lib.cera_hip_ctx_set_decode_copies(self.h, 1 if enabled else 0))

    def device_info(self):
        name = C.create_string_buffer(256)
        cu, hbm = C.c_uint32(), C.c_uint64()
        self.check(self.lib.cera_hip_device_info(self.h, name, C.byref(cu), C.byref(hbm)))
        return name.value.decode(), cu.value, hbm.value

    # -- device memory
    def malloc(self, nbytes: int) -> int:
        p = C.c_void_p()
        self.check(self.lib.cera_hip_malloc(self.h, nbytes, C.byref(p)))
        return p.value

    def free(self, dev: int):
        self.check(self.lib.cera_hip_free(self.h, dev))

    def upload(self, dev: int, arr: np.ndarray):
        arr = np.ascontiguousarray(arr)
        self.check(self.lib.cera_hip_upload(self.h, dev, _p(arr), arr.nbytes))

    def to_device(self, arr: np.ndarray) -> int:
        arr = np.ascontiguousarray(arr)
        d = self.malloc(arr.nbytes)
        self.upload(d, arr)
        return d

    def download(self, dev: int, shape, dtype) -> np.ndarray:
        out = np.empty(shape, dtype)
        self.check(self.lib.cera_hip_download(self.h, _p(out), dev, out.nbytes))
        return out

    # -- events
    def event(self) -> int:
        e = C.c_void_p()
        self.check(self.lib.cera_hip_event_create(self.h, C.byref(e)))
        return e.value

    def record(self, ev: int):
        self.check(self.lib.cera_hip_event_record(self.h, ev))

    def elapsed_ms(self, a: int, b: int) -> float:
        ms = C.c_float()
        self.check(self.lib.cera_hip_event_elapsed_ms(self.h, a, b, C.byref(ms)))
        return ms.value

    def event_destroy(self, ev: int):
        self.lib.cera_hip_event_destroy(ev)

    # -- weights
    def tensor_upload(self, ggml_type: int, m: int, k: int, blocks: np.ndarray) -> int:
        t = make_tensor(ggml_type, m, k, blocks)
        h = C.c_void_p()
        self.check(self.lib.cera_hip_tensor_upload(self.h, C.byref(t), C.byref(h)))
        return h.value

    def tensor_clone(self, dt: int) -> int:
        h = C.c_void_p()
        self.check(self.lib.cera_hip_tensor_clone(self.h, dt, C.byref(h)))
        return h.value

    def tensor_free(self, dt: int):
        self.lib.cera_hip_tensor_free(self.h, dt)

    # -- kernel level, host buffers
    def quantize_q8_0(self, x: np.ndarray):
        x = np.ascontiguousarray(x, np.float32).reshape(-1)
        k = x.size
        scales = np.empty(max(k // 32, 0), np.float32)
        quants = np.empty(k, np.int8)
        self.check(self.lib.cera_hip_quantize_q8_0(self.h, _p(x), k, _p(scales), _p(quants)))
        return scales, quants

    def gemv(self, ggml_type: int, blocks: np.ndarray, x: np.ndarray, m: int, k: int, debug: bool = False):
        t = make_tensor(ggml_type, m, k, blocks)
        x = np.ascontiguousarray(x, np.float32)
        y = np.empty(m, np.float32)
        if not debug:
            self.check(self.lib.cera_hip_gemv(self.h, C.byref(t), _p(x), _p(y), None, None))
            return y
        nd = k // 16 if ggml_type == Q6_K else k // 32
        dots = np.zeros((m, nd), np.int32)
        asums = np.zeros(nd, np.int32)
        self.check(self.lib.cera_hip_gemv(self.h, C.byref(t), _p(x), _p(y), _p(dots), _p(asums)))
        return y, dots, asums

    def gemv_add_dev(self, ggml_type: int, blocks: np.ndarray, x: np.ndarray, resid: np.ndarray, m: int, k: int) -> np.ndarray:
        """resid + W.Q8_0(x) the way the decode step launches it (a quantize op, then a GEMV op with a residual)."""
        dt = self.tensor_upload(ggml_type, m, k, blocks)
        d_x = self.to_device(np.ascontiguousarray(x, np.float32))
        d_r = self.to_device(np.ascontiguousarray(resid, np.float32))
        d_s, d_q, d_y = self.malloc(max(k // 32, 1) * 4), self.malloc(k), self.malloc(m * 4)
        ops = (DecodeOp * 2)(DecodeOp(kind=DecodeOp.QUANT, n=k, x=d_x, out_q=d_q, out_s=d_s),
                             DecodeOp(kind=DecodeOp.GEMV, w=dt, xs=d_s, xq=d_q, resid=d_r, y=d_y))
        try:
            self.check(self.lib.cera_hip_decode_ops_dev(self.h, ops, 2))
            return self.download(d_y, m, np.float32)
        finally:
            for d in (d_x, d_r, d_s, d_q, d_y):
                self.free(d)
            self.tensor_free(dt)

    def gemv_store_dev(self, ggml_type: int, blocks: np.ndarray, x: np.ndarray, m: int, k: int) -> np.ndarray:
        """W.Q8_0(x) the way the decode step launches its vocabulary head (a quantize op, then a GEMV op without a residual)."""
        dt = self.tensor_upload(ggml_type, m, k, blocks)
        d_x = self.to_device(np.ascontiguousarray(x, np.float32))
        d_s, d_q, d_y = self.malloc(max(k // 32, 1) * 4), self.malloc(k), self.malloc(m * 4)
        ops = (DecodeOp * 2)(DecodeOp(kind=DecodeOp.QUANT, n=k, x=d_x, out_q=d_q, out_s=d_s),
                             DecodeOp(kind=DecodeOp.GEMV, w=dt, xs=d_s, xq=d_q, y=d_y))
        try:
            self.check(self.lib.cera_hip_decode_ops_dev(self.h, ops, 2))
            return self.download(d_y, m, np.float32)
        finally:
            for d in (d_x, d_s, d_q, d_y):
                self.free(d)
            self.tensor_free(dt)

    def gemm(self, ggml_type: int, blocks: np.ndarray, x: np.ndarray, m: int, n: int, k: int) -> np.ndarray:
        t = make_tensor(ggml_type, m, k, blocks)
        x = np.ascontiguousarray(x, np.float32).reshape(n, k)
        out = np.empty((m, n), np.float32)
        self.check(self.lib.cera_hip_gemm(self.h, C.byref(t), _p(x), n, _p(out)))
        return out

    def gemm_block_dots(self, ggml_type: int, blocks: np.ndarray, x: np.ndarray, m: int, n: int, k: int):
        """(dots, out): dots int32 [m][n][k/32], or for Q6_K float32 [m][n][k/16] (the f16 MFMA's results)."""
        t = make_tensor(ggml_type, m, k, blocks)
        x = np.ascontiguousarray(x, np.float32).reshape(n, k)
        per = k // 16 if ggml_type == Q6_K else k // 32
        dots = np.zeros((m, n, per), np.int32)
        out = np.empty((m, n), np.float32)
        self.check(self.lib.cera_hip_gemm_block_dots(self.h, C.byref(t), _p(x), n, _p(dots), _p(out)))
        return (dots.view(np.float32) if ggml_type == Q6_K else dots), out

    def attn_decode(self, q, k, v, n_heads, n_kv_heads, head_dim, seq_len, scale, n_splits=0) -> np.ndarray:
        q = np.ascontiguousarray(q, np.float32)
        k = np.ascontiguousarray(k, np.float32)
        v = np.ascontiguousarray(v, np.float32)
        out = np.empty(n_heads * head_dim, np.float32)
        self.check(self.lib.cera_hip_attn_decode(self.h, _p(q), _p(k), _p(v), n_heads, n_kv_heads, head_dim, seq_len,
                                                 scale, n_splits, _p(out)))
        return out

    def attn_prefill(self, q, k, v, n_heads, n_kv_heads, head_dim, start_pos, n_queries, scale) -> np.ndarray:
        q = np.ascontiguousarray(q, np.float32)
        k = np.ascontiguousarray(k, np.float32)
        v = np.ascontiguousarray(v, np.float32)
        out = np.empty(n_queries * n_heads * head_dim, np.float32)
        self.check(self.lib.cera_hip_attn_prefill(self.h, _p(q), _p(k), _p(v), n_heads, n_kv_heads, head_dim, start_pos,
                                                  n_queries, scale, _p(out)))
        return out.reshape(n_queries, n_heads * head_dim)

    def gemv_nb(self, ggml_type: int, blocks: np.ndarray, x: np.ndarray, m: int, k: int) -> np.ndarray:
        """x [n][k] -> y [n][m] through the multi-token GEMV."""
        t = make_tensor(ggml_type, m, k, blocks)
        x = np.ascontiguousarray(x, np.float32).reshape(-1, k)
        y = np.empty((x.shape[0], m), np.float32)
        self.check(self.lib.cera_hip_gemv_nb(self.h, C.byref(t), _p(x), x.shape[0], _p(y)))
        return y

    def gemv_pair(self, type_a, wa, ma, type_b, wb, mb, x, k):
        ta, tb = make_tensor(type_a, ma, k, wa), make_tensor(type_b, mb, k, wb)
        x = np.ascontiguousarray(x, np.float32)
        ya, yb = np.empty(ma, np.float32), np.empty(mb, np.float32)
        self.check(self.lib.cera_hip_gemv_pair(self.h, C.byref(ta), C.byref(tb), _p(x), _p(ya), _p(yb)))
        return ya, yb

    def gemm_pair(self, type_a, wa, ma, type_b, wb, mb, x, n, k):
        """Two matrices of one type against the same n activation rows in one launch; token-major outputs."""
        ta, tb = make_tensor(type_a, ma, k, wa), make_tensor(type_b, mb, k, wb)
        x = np.ascontiguousarray(x, np.float32).reshape(n, k)
        oa, ob = np.empty((n, ma), np.float32), np.empty((n, mb), np.float32)
        self.check(self.lib.cera_hip_gemm_pair(self.h, C.byref(ta), C.byref(tb), _p(x), n, _p(oa), _p(ob)))
        return oa, ob

    def gemm_swiglu(self, type_id, w_gate, w_up, m, x, n, k):
        """Q8_0(silu(gate.x) * (up.x)) per token row: (quants [n][m] int8, scales [n][m/32], fused?)."""
        tg, tu = make_tensor(type_id, m, k, w_gate), make_tensor(type_id, m, k, w_up)
        x = np.ascontiguousarray(x, np.float32).reshape(n, k)
        q, sc = np.empty((n, m), np.int8), np.empty((n, m // 32), np.float32)
        fused = C.c_int(-1)
        self.check(self.lib.cera_hip_gemm_swiglu(self.h, C.byref(tg), C.byref(tu), _p(x), n, _p(q), _p(sc), C.byref(fused)))
        return q, sc, bool(fused.value)

    def gemm_swiglu_f16(self, type_id, w_gate, w_up, m, x, n, k):
        """gemm_swiglu plus the quants as the f16 words a Q6_K down projection reads: (quants, scales, halves [n][m] uint16, fused?)."""
        tg, tu = make_tensor(type_id, m, k, w_gate), make_tensor(type_id, m, k, w_up)
        x = np.ascontiguousarray(x, np.float32).reshape(n, k)
        q, sc, hv = np.empty((n, m), np.int8), np.empty((n, m // 32), np.float32), np.empty((n, m), np.uint16)
        fused = C.c_int(-1)
        self.check(self.lib.cera_hip_gemm_swiglu_f16(self.h, C.byref(tg), C.byref(tu), _p(x), n, _p(q), _p(sc), _p(hv), C.byref(fused)))
        return q, sc, hv, bool(fused.value)

    def attn_f16kv(self, q, k, v, n_heads, n_kv_heads, head_dim, start_pos, n_queries, scale, n_splits=0) -> np.ndarray:
        """Attention over an f16 KV cache: k, v (f32) are narrowed to half before the upload."""
        q = np.ascontiguousarray(q, np.float32)
        k = np.ascontiguousarray(k, np.float32)
        v = np.ascontiguousarray(v, np.float32)
        out = np.empty(n_queries * n_heads * head_dim, np.float32)
        self.check(self.lib.cera_hip_attn_f16kv(self.h, _p(q), _p(k), _p(v), n_heads, n_kv_heads, head_dim, start_pos,
                                                n_queries, scale, n_splits, _p(out)))
        return out.reshape(n_queries, n_heads * head_dim)

    def ffn_gate_up_fused(self, w_gate, w_up, m, k, x, norm_w, eps, ggml_type: int = Q4_K):
        """Q8_0(silu(gate.n) * (up.n)), n = Q8_0(rmsnorm(x, norm_w)): (quants [m], scales [m/32])."""
        tg, tu = make_tensor(ggml_type, m, k, w_gate), make_tensor(ggml_type, m, k, w_up)
        x = np.ascontiguousarray(x, np.float32); nw = np.ascontiguousarray(norm_w, np.float32)
        q, sc = np.empty(m, np.int8), np.empty(m // 32, np.float32)
        self.check(self.lib.cera_hip_ffn_gate_up_fused(self.h, C.byref(tg), C.byref(tu), _p(x), _p(nw), eps, _p(q), _p(sc)))
        return q, sc

    def qkv_fused(self, type_a, wa, ma, type_b, wb, mb, k, x, norm_w, eps):
        ta = make_tensor(type_a, ma, k, wa)
        tb = make_tensor(type_b, mb, k, wb) if wb is not None else None
        x = np.ascontiguousarray(x, np.float32); nw = np.ascontiguousarray(norm_w, np.float32)
        ya = np.empty(ma, np.float32); yb = np.empty(mb, np.float32) if wb is not None else None
        self.check(self.lib.cera_hip_qkv_fused(self.h, C.byref(ta), C.byref(tb) if tb is not None else None, _p(x), _p(nw), eps,
                                               _p(ya), _p(yb) if yb is not None else None))
        return ya, yb

    # -- the decode step's fused kernels
    def rmsnorm_q8_0(self, x, w, eps):
        """(normed f32, Q8_0 scales, Q8_0 quants) from the decode step's one-launch norm + quantize."""
        x = np.ascontiguousarray(x, np.float32)
        w = np.ascontiguousarray(w, np.float32)
        y = np.empty_like(x)
        scales = np.empty(x.size // 32, np.float32)
        quants = np.empty(x.size, np.int8)
        self.check(self.lib.cera_hip_rmsnorm_q8_0(self.h, _p(x), _p(w), x.size, eps, _p(y), _p(scales), _p(quants)))
        return y, scales, quants

    def attn_decode_step(self, q, k_new, v_new, k_cache, v_cache, n_heads, n_kv_heads, head_dim, pos, rope_base,
                         norm=True, freq_factors=None, scale=None, kv_f16=False):
        """One decode layer's attention step: (out, out_scales, out_quants, appended k row, appended v row)."""
        q = np.ascontiguousarray(q, np.float32); k_new = np.ascontiguousarray(k_new, np.float32)
        v_new = np.ascontiguousarray(v_new, np.float32)
        kc = np.ascontiguousarray(k_cache, np.float32); vc = np.ascontiguousarray(v_cache, np.float32)
        ff = None if freq_factors is None else np.ascontiguousarray(freq_factors, np.float32)
        q_dim, kv_dim = n_heads * head_dim, n_kv_heads * head_dim
        out = np.empty(q_dim, np.float32); sc = np.empty(q_dim // 32, np.float32); qq = np.empty(q_dim, np.int8)
        k_row = np.empty(kv_dim, np.float32); v_row = np.empty(kv_dim, np.float32)
        scale = float(scale if scale is not None else 1.0 / np.sqrt(head_dim))
        self.check(self.lib.cera_hip_attn_decode_step(
            self.h, _p(q), _p(k_new), _p(v_new), _p(kc) if kc.size else None, _p(vc) if vc.size else None, n_heads,
            n_kv_heads, head_dim, pos, rope_base, 1 if norm else 0, None if ff is None else _p(ff), scale,
            1 if kv_f16 else 0, _p(out), _p(sc), _p(qq), _p(k_row), _p(v_row)))
        return out, sc, qq, k_row, v_row

    # -- reference-order verification kernels (bit-identical to the CPU AVX2 path)
    def gemv_reference_order(self, ggml_type: int, blocks: np.ndarray, x: np.ndarray, m: int, k: int) -> np.ndarray:
        t = make_tensor(ggml_type, m, k, blocks)
        x = np.ascontiguousarray(x, np.float32)
        y = np.empty(m, np.float32)
        self.check(self.lib.cera_hip_gemv_reference_order(self.h, C.byref(t), _p(x), _p(y)))
        return y

    def attn_decode_reference_order(self, q, k, v, n_heads, n_kv_heads, head_dim, seq_len, scale) -> np.ndarray:
        q = np.ascontiguousarray(q, np.float32)
        k = np.ascontiguousarray(k, np.float32)
        v = np.ascontiguousarray(v, np.float32)
        out = np.empty(n_heads * head_dim, np.float32)
        self.check(self.lib.cera_hip_attn_decode_reference_order(self.h, _p(q), _p(k), _p(v), n_heads, n_kv_heads, head_dim,
                                                                 seq_len, scale, _p(out)))
        return out

    def gemm_reference_order(self, ggml_type: int, blocks: np.ndarray, x: np.ndarray, m: int, k: int,
                             x86_repack: bool = True) -> np.ndarray:
        """out[m][n] = W . Q8_0(x[n][k]) in the order of the x86 host's batched prefill route."""
        t = make_tensor(ggml_type, m, k, blocks)
        x = np.ascontiguousarray(x, np.float32).reshape(-1, k)
        out = np.empty((m, x.shape[0]), np.float32)
        self.check(self.lib.cera_hip_gemm_reference_order(self.h, C.byref(t), _p(x), x.shape[0], 1 if x86_repack else 0, _p(out)))
        return out

    def flash_attn_reference_order(self, q, k, v, n_heads, n_kv_heads, head_dim, start_pos, scale) -> np.ndarray:
        """q [n][n_heads * head_dim]; k, v time-major [start_pos + n][n_kv_heads * head_dim]."""
        q = np.ascontiguousarray(q, np.float32).reshape(-1, n_heads * head_dim)
        k = np.ascontiguousarray(k, np.float32)
        v = np.ascontiguousarray(v, np.float32)
        out = np.empty_like(q)
        self.check(self.lib.cera_hip_flash_attn_reference_order(self.h, _p(q), _p(k), _p(v), q.shape[0], n_heads, n_kv_heads,
                                                                head_dim, start_pos, scale, _p(out)))
        return out

    def rmsnorm_reference_order(self, x, w, eps) -> np.ndarray:
        x = np.ascontiguousarray(x, np.float32)
        w = np.ascontiguousarray(w, np.float32)
        y = np.empty_like(x)
        self.check(self.lib.cera_hip_rmsnorm_reference_order(self.h, _p(x), _p(w), x.size, eps, _p(y)))
        return y

    def rmsnorm(self, x, w, eps) -> np.ndarray:
        x = np.ascontiguousarray(x, np.float32)
        w = np.ascontiguousarray(w, np.float32)
        y = np.empty_like(x)
        self.check(self.lib.cera_hip_rmsnorm(self.h, _p(x), _p(w), x.size, eps, _p(y)))
        return y

    def silu_mul(self, gate, up) -> np.ndarray:
        g = np.ascontiguousarray(gate, np.float32)
        u = np.ascontiguousarray(up, np.float32)
        y = np.empty_like(g)
        self.check(self.lib.cera_hip_silu_mul(self.h, _p(g), _p(u), g.size, _p(y)))
        return y

    def rope(self, q, k, pos, n_heads, n_kv_heads, head_dim, base, norm=True, freq_factors=None):
        q2 = np.array(q, np.float32, copy=True).reshape(-1)
        k2 = np.array(k, np.float32, copy=True).reshape(-1)
        ff = None if freq_factors is None else np.ascontiguousarray(freq_factors, np.float32)
        self.check(self.lib.cera_hip_rope(self.h, _p(q2), _p(k2), pos, n_heads, n_kv_heads, head_dim, base,
                                          1 if norm else 0, None if ff is None else _p(ff)))
        return q2, k2

    def argmax(self, logits) -> int:
        l = np.ascontiguousarray(logits, np.float32)
        idx = C.c_uint32()
        self.check(self.lib.cera_hip_argmax(self.h, _p(l) if l.size else None, l.size, C.byref(idx)))
        return idx.value

    def dequantize_row(self, ggml_type, blocks, m, k, row) -> np.ndarray:
        t = make_tensor(ggml_type, m, k, blocks)
        out = np.empty(k, np.float32)
        self.check(self.lib.cera_hip_dequantize_row(self.h, C.byref(t), row, _p(out)))
        return out


class Model:
    """cera_hip_model: the `Model`-trait surface over a device-resident llama.

    ``weights``: name -> (ggml_type, m, k, uint8 blocks) for matrices and
    name -> float32 array for norm vectors, GGUF tensor names.
    """

    def __init__(self, ctx: Context, cfg: dict, weights: dict):
        self.ctx = ctx
        c = make_config(cfg)
        self.cfg = dict(cfg)
        keep = []
        rf = weights.get("rope_freqs.weight")
        if rf is not None:
            rf = np.ascontiguousarray(rf, np.float32)
            keep.append(rf)
            c.rope_freqs = rf.ctypes.data
        layers = (Layer * c.n_layers)()
        for i in range(c.n_layers):
            L = layers[i]
            for nm in ("attn_norm", "ffn_norm"):
                a = np.ascontiguousarray(weights[f"blk.{i}.{nm}.weight"], np.float32)
                keep.append(a)
                setattr(L, nm, a.ctypes.data)
            for nm in ("attn_q", "attn_k", "attn_v", "attn_output", "ffn_gate", "ffn_up", "ffn_down"):
                dt, m, k, arr = weights[f"blk.{i}.{nm}.weight"]
                t = make_tensor(dt, m, k, arr)
                keep.append(t)
                setattr(L, nm, t)
            for nm, key in (("q_bias", "attn_q.bias"), ("k_bias", "attn_k.bias"), ("v_bias", "attn_v.bias"),
                            ("q_norm", "attn_q_norm.weight"), ("k_norm", "attn_k_norm.weight")):
                a = weights.get(f"blk.{i}.{key}")
                if a is not None:
                    a = np.ascontiguousarray(a, np.float32)
                    keep.append(a)
                setattr(L, nm, a.ctypes.data if a is not None else None)
        dt, m, k, arr = weights["token_embd.weight"]
        embd = make_tensor(dt, m, k, arr)
        outp = None
        if "output.weight" in weights:
            dt, m, k, arr = weights["output.weight"]
            outp = make_tensor(dt, m, k, arr)
        onorm = np.ascontiguousarray(weights["output_norm.weight"], np.float32)
        h = C.c_void_p()
        st = ctx.lib.cera_hip_model_create(ctx.h, C.byref(c), C.byref(embd), C.byref(outp) if outp is not None else None,
                                           onorm.ctypes.data, layers, C.byref(h))
        ctx.check(st)
        self.h = h
        self.vocab = c.vocab
        self.hidden = c.hidden

    @property
    def seq_len(self) -> int:
        return int(self.ctx.lib.cera_hip_seq_len(self.h))

    @property
    def memory_bytes(self) -> int:
        return int(self.ctx.lib.cera_hip_memory_bytes(self.h))

    def drop_decode_copies(self) -> int:
        """Free every decode copy of the model; returns the bytes given back."""
        freed = C.c_uint64()
        self.ctx.check(self.ctx.lib.cera_hip_drop_decode_copies(self.h, C.addressof(freed)))
        return int(freed.value)

    def forward(self, token: int, pos: int) -> np.ndarray:
        logits = np.empty(self.vocab, np.float32)
        self.ctx.check(self.ctx.lib.cera_hip_forward(self.h, token, pos, _p(logits)))
        return logits

    def forward_greedy(self, token: int, pos: int) -> int:
        nxt = C.c_uint32()
        self.ctx.check(self.ctx.lib.cera_hip_forward_greedy(self.h, token, pos, C.byref(nxt)))
        return nxt.value

    def forward_prefill(self, tokens, start_pos: int) -> np.ndarray:
        t = np.ascontiguousarray(tokens, np.uint32)
        logits = np.empty(self.vocab, np.float32)
        self.ctx.check(self.ctx.lib.cera_hip_forward_prefill(self.h, _p(t), t.size, start_pos, _p(logits)))
        return logits

    def forward_prefill_logits_all(self, tokens, start_pos: int) -> np.ndarray:
        t = np.ascontiguousarray(tokens, np.uint32)
        out = np.empty((t.size, self.vocab), np.float32)
        self.ctx.check(self.ctx.lib.cera_hip_forward_prefill_logits_all(self.h, _p(t) if t.size else None, t.size, start_pos,
                                                                        _p(out)))
        return out

    def set_reference_order(self, on=True):
        """Switch to (or from) the reference-order verification route; needs an empty cache.
        True / 1: prefill token by token; 2: prompts of more than one token in the x86 host's
        batched order (forward_prefill_batched with the repacked 8x8 kernels and the AVX2 flash
        attention)."""
        self.ctx.check(self.ctx.lib.cera_hip_set_reference_order(self.h, int(on)))

    @property
    def reference_order(self) -> int:
        return int(self.ctx.lib.cera_hip_reference_order(self.h))

    def configure_kv(self, f16: bool):
        self.ctx.check(self.ctx.lib.cera_hip_configure_kv(self.h, 1 if f16 else 0))

    @property
    def kv_f16(self) -> bool:
        return self.ctx.lib.cera_hip_kv_type(self.h) == 1

    def shift_kv(self, n_keep: int, shift: int):
        self.ctx.check(self.ctx.lib.cera_hip_shift_kv(self.h, n_keep, shift))

    def write_kv(self, layer: int, k: np.ndarray, v: np.ndarray):
        k = np.ascontiguousarray(k, np.float32); v = np.ascontiguousarray(v, np.float32)
        kv_dim = self.cfg["n_kv_heads"] * self.cfg["head_dim"]
        assert k.size == v.size and k.size % kv_dim == 0
        self.ctx.check(self.ctx.lib.cera_hip_write_kv(self.h, layer, _p(k) if k.size else None,
                                                      _p(v) if v.size else None, k.size // kv_dim))

    def set_seq_len(self, n: int):
        self.ctx.check(self.ctx.lib.cera_hip_set_seq_len(self.h, n))

    def truncate_kv(self, n: int):
        self.ctx.check(self.ctx.lib.cera_hip_truncate_kv(self.h, n))

    def read_kv(self, layer: int):
        n = self.seq_len * self.cfg["n_kv_heads"] * self.cfg["head_dim"]
        k = np.empty(n, np.float32)
        v = np.empty(n, np.float32)
        self.ctx.check(self.ctx.lib.cera_hip_read_kv(self.h, layer, _p(k), _p(v)))
        return k, v

    def read_hidden(self) -> np.ndarray:
        h = np.empty(self.hidden, np.float32)
        self.ctx.check(self.ctx.lib.cera_hip_read_hidden(self.h, _p(h)))
        return h

    def close(self):
        if getattr(self, "h", None):
            self.ctx.lib.cera_hip_model_destroy(self.h)
            self.h = None
