//! Raw bindings of `libcera_hip.so` — the AMD MI355X (gfx950) compute backend for cera's dense
//! transformer decode / prefill hot path. One declaration per entry point of the C header
//! `include/cera_hip.h` of the backend, in the header's order; the header documents each one and
//! names the cera interface it stands in for.
//!
//! Conventions of the library (see the header for the full text):
//! * every fallible call returns a [`cera_hip_status`]; the message of the last failure on a
//!   context comes from [`cera_hip_last_error`]; nothing aborts or unwinds across the boundary;
//! * "host" pointers are caller-owned CPU memory borrowed for the duration of the call, "dev"
//!   pointers come from [`cera_hip_malloc`] on the same context;
//! * calls on one context are serialised by the library, a model additionally by its own lock.
#![allow(non_camel_case_types)]
#![allow(clippy::too_many_arguments)]

use std::os::raw::{c_char, c_int, c_void};

/// Device, stream and scratch memory.
#[repr(C)]
pub struct cera_hip_ctx {
    _opaque: [u8; 0],
}
/// Device-resident weights, KV cache and sequence length of one model.
#[repr(C)]
pub struct cera_hip_model {
    _opaque: [u8; 0],
}
/// One weight matrix resident in HBM.
#[repr(C)]
pub struct cera_hip_dtensor {
    _opaque: [u8; 0],
}
/// A HIP event on the context's stream.
#[repr(C)]
pub struct cera_hip_event {
    _opaque: [u8; 0],
}

/// `cera_hip_status` of the header (a C enum: an `int`).
pub type cera_hip_status = c_int;
pub const CERA_HIP_OK: cera_hip_status = 0;
/// HIP runtime error (the message carries the HIP string).
pub const CERA_HIP_ERR_DEVICE: cera_hip_status = 1;
/// Device or host allocation failed.
pub const CERA_HIP_ERR_OOM: cera_hip_status = 2;
/// No kernel for this GGML type: refused, never skipped.
pub const CERA_HIP_ERR_UNSUPPORTED_DTYPE: cera_hip_status = 3;
/// Size / shape / alignment does not fit the kernel.
pub const CERA_HIP_ERR_SHAPE: cera_hip_status = 4;
/// `pos` / `start_pos` differs from the current sequence length.
pub const CERA_HIP_ERR_POSITION: cera_hip_status = 5;
/// Null pointer or out-of-range scalar.
pub const CERA_HIP_ERR_ARGUMENT: cera_hip_status = 6;

// GGML type ids as cera maps them (cera/src/gguf.rs).
pub const CERA_HIP_F32: u32 = 0;
pub const CERA_HIP_F16: u32 = 1;
pub const CERA_HIP_Q4_0: u32 = 2;
pub const CERA_HIP_Q4_1: u32 = 3;
pub const CERA_HIP_Q8_0: u32 = 8;
pub const CERA_HIP_Q4_K: u32 = 12;
pub const CERA_HIP_Q5_K: u32 = 13;
pub const CERA_HIP_Q6_K: u32 = 14;
pub const CERA_HIP_BF16: u32 = 30;

/// KV cache element types for [`cera_hip_configure_kv`].
pub const CERA_HIP_KV_F32: u32 = 0;
pub const CERA_HIP_KV_F16: u32 = 1;

/// Size of the fixed per-GPU workspace behind [`cera_hip_attn_decode_dev_noalloc`].
pub const CERA_HIP_NOALLOC_WORKSPACE_BYTES: u32 = 4 << 20;

/// Kinds of a [`cera_hip_decode_op`].
pub const CERA_HIP_OP_GEMV: u32 = 0;
pub const CERA_HIP_OP_NORM_GEMV: u32 = 1;
pub const CERA_HIP_OP_NORM_GATE_UP: u32 = 2;
pub const CERA_HIP_OP_NORM_QUANT: u32 = 3;
pub const CERA_HIP_OP_QUANT: u32 = 4;

/// A weight matrix as cera resolves it from a GGUF: `WeightRef {dtype, m, k}` plus the mmap
/// slice. `m` output rows, `k` inner dimension; `data` is `m` rows of native GGML blocks (host).
#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct cera_hip_tensor {
    pub ggml_type: u32,
    pub _reserved: u32,
    pub m: u64,
    pub k: u64,
    pub data: *const c_void,
    pub nbytes: u64,
}

/// Per-layer weights. The norm / bias vectors are host `f32`; the optional ones are null when
/// the architecture has none (biases: Qwen2, per-head QK norms: Qwen3).
#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct cera_hip_layer {
    pub attn_norm: *const f32,
    pub ffn_norm: *const f32,
    pub attn_q: cera_hip_tensor,
    pub attn_k: cera_hip_tensor,
    pub attn_v: cera_hip_tensor,
    pub attn_output: cera_hip_tensor,
    pub ffn_gate: cera_hip_tensor,
    pub ffn_up: cera_hip_tensor,
    pub ffn_down: cera_hip_tensor,
    pub q_bias: *const f32,
    pub k_bias: *const f32,
    pub v_bias: *const f32,
    pub q_norm: *const f32,
    pub k_norm: *const f32,
}

/// `ModelConfig` + attention dimensions.
#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct cera_hip_config {
    pub n_layers: u32,
    pub hidden: u32,
    pub ffn: u32,
    pub n_heads: u32,
    pub n_kv_heads: u32,
    pub head_dim: u32,
    pub vocab: u32,
    pub max_seq_len: u32,
    /// 0 = NEOX (split halves), 1 = NORM (interleaved pairs).
    pub rope_type: u32,
    pub rope_theta: f32,
    pub rms_eps: f32,
    pub embed_scale: f32,
    pub residual_scale: f32,
    /// 0 selects `1 / sqrt(head_dim)`.
    pub attn_scale: f32,
    /// Logits are divided by this; 1 = off.
    pub logit_scale: f32,
    /// Nullable, `f32[head_dim / 2]`.
    pub rope_freqs: *const f32,
}

/// One launch of [`cera_hip_gemv_seq_dev`]; all pointers are device pointers.
#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct cera_hip_gemv_op {
    pub w: *const cera_hip_dtensor,
    /// Nullable: the fused FFN pair `silu(w.x) * (w2.x)`.
    pub w2: *const cera_hip_dtensor,
    pub xs: *const f32,
    pub xq: *const i8,
    pub y: *mut f32,
}

/// One launch of [`cera_hip_decode_ops_dev`]; all pointers are device pointers.
#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct cera_hip_decode_op {
    pub kind: u32,
    pub n: u32,
    pub w: *const cera_hip_dtensor,
    pub w2: *const cera_hip_dtensor,
    pub x: *const f32,
    pub norm_w: *const f32,
    pub eps: f32,
    pub xs: *const f32,
    pub xq: *const i8,
    pub resid: *const f32,
    pub y: *mut f32,
    pub y2: *mut f32,
    pub out_s: *mut f32,
    pub out_q: *mut i8,
}

unsafe extern "C" {
pub fn cera_hip_ctx_create(
        device: c_int,
        hsaco_path: *const c_char,
        out: *mut *mut cera_hip_ctx,
    ) -> cera_hip_status;
    pub fn cera_hip_ctx_destroy(ctx: *mut cera_hip_ctx);
    pub fn cera_hip_ctx_set_decode_copies(ctx: *mut cera_hip_ctx, enabled: c_int) -> cera_hip_status;
    pub fn cera_hip_decode_copy_reserve_bytes(cfg: *const cera_hip_config) -> u64;
    pub fn cera_hip_decode_copy_plan(
        copy_bytes: *const u64,
        n: u32,
        free_bytes: u64,
        reserve_bytes: u64,
        take: *mut u8,
    ) -> u64;
    pub fn cera_hip_last_error(ctx: *const cera_hip_ctx) -> *const c_char;
    pub fn cera_hip_sync(ctx: *mut cera_hip_ctx) -> cera_hip_status;
    pub fn cera_hip_device_info(
        ctx: *mut cera_hip_ctx,
        name256: *mut c_char,
        n_cu: *mut u32,
        hbm_bytes: *mut u64,
    ) -> cera_hip_status;
    pub fn cera_hip_malloc(
        ctx: *mut cera_hip_ctx,
        nbytes: u64,
        dev_out: *mut *mut c_void,
    ) -> cera_hip_status;
    pub fn cera_hip_free(ctx: *mut cera_hip_ctx, dev: *mut c_void) -> cera_hip_status;
    pub fn cera_hip_upload(
        ctx: *mut cera_hip_ctx,
        dev_dst: *mut c_void,
        host_src: *const c_void,
        nbytes: u64,
    ) -> cera_hip_status;
    pub fn cera_hip_download(
        ctx: *mut cera_hip_ctx,
        host_dst: *mut c_void,
        dev_src: *const c_void,
        nbytes: u64,
    ) -> cera_hip_status;
    pub fn cera_hip_copy_dev(
        ctx: *mut cera_hip_ctx,
        dev_dst: *mut c_void,
        dev_src: *const c_void,
        nbytes: u64,
    ) -> cera_hip_status;
    pub fn cera_hip_copy_kernel(
        ctx: *mut cera_hip_ctx,
        dev_dst: *mut c_void,
        dev_src: *const c_void,
        nbytes: u64,
    ) -> cera_hip_status;
    pub fn cera_hip_event_create(
        ctx: *mut cera_hip_ctx,
        out: *mut *mut cera_hip_event,
    ) -> cera_hip_status;
    pub fn cera_hip_event_destroy(event: *mut cera_hip_event);
    pub fn cera_hip_event_record(
        ctx: *mut cera_hip_ctx,
        event: *mut cera_hip_event,
    ) -> cera_hip_status;
    pub fn cera_hip_event_elapsed_ms(
        ctx: *mut cera_hip_ctx,
        start: *mut cera_hip_event,
        stop: *mut cera_hip_event,
        ms: *mut f32,
    ) -> cera_hip_status;
    pub fn cera_hip_tensor_upload(
        ctx: *mut cera_hip_ctx,
        t: *const cera_hip_tensor,
        out: *mut *mut cera_hip_dtensor,
    ) -> cera_hip_status;
    pub fn cera_hip_tensor_clone(
        ctx: *mut cera_hip_ctx,
        src: *const cera_hip_dtensor,
        out: *mut *mut cera_hip_dtensor,
    ) -> cera_hip_status;
    pub fn cera_hip_tensor_free(ctx: *mut cera_hip_ctx, tensor: *mut cera_hip_dtensor);
    pub fn cera_hip_tensor_nbytes(tensor: *const cera_hip_dtensor) -> u64;
    pub fn cera_hip_quantize_q8_0(
        ctx: *mut cera_hip_ctx,
        x: *const f32,
        k: u64,
        scales: *mut f32,
        quants: *mut i8,
    ) -> cera_hip_status;
    pub fn cera_hip_gemv(
        ctx: *mut cera_hip_ctx,
        w: *const cera_hip_tensor,
        x: *const f32,
        y: *mut f32,
        dbg_block_dots: *mut i32,
        dbg_block_asums: *mut i32,
    ) -> cera_hip_status;
    pub fn cera_hip_gemv_nb(
        ctx: *mut cera_hip_ctx,
        w: *const cera_hip_tensor,
        x: *const f32,
        n: u32,
        y: *mut f32,
    ) -> cera_hip_status;
    pub fn cera_hip_gemv_pair(
        ctx: *mut cera_hip_ctx,
        a: *const cera_hip_tensor,
        b: *const cera_hip_tensor,
        x: *const f32,
        ya: *mut f32,
        yb: *mut f32,
    ) -> cera_hip_status;
    pub fn cera_hip_gemm(
        ctx: *mut cera_hip_ctx,
        w: *const cera_hip_tensor,
        x: *const f32,
        n: u64,
        out: *mut f32,
    ) -> cera_hip_status;
    pub fn cera_hip_gemm_block_dots(
        ctx: *mut cera_hip_ctx,
        w: *const cera_hip_tensor,
        x: *const f32,
        n: u64,
        dots: *mut i32,
        out: *mut f32,
    ) -> cera_hip_status;
    pub fn cera_hip_gemm_pair(
        ctx: *mut cera_hip_ctx,
        a: *const cera_hip_tensor,
        b: *const cera_hip_tensor,
        x: *const f32,
        n: u64,
        out_a: *mut f32,
        out_b: *mut f32,
    ) -> cera_hip_status;
    pub fn cera_hip_gemm_swiglu(
        ctx: *mut cera_hip_ctx,
        gate: *const cera_hip_tensor,
        up: *const cera_hip_tensor,
        x: *const f32,
        n: u64,
        quants: *mut i8,
        scales: *mut f32,
        fused: *mut c_int,
    ) -> cera_hip_status;
    pub fn cera_hip_gemm_swiglu_f16(
        ctx: *mut cera_hip_ctx,
        gate: *const cera_hip_tensor,
        up: *const cera_hip_tensor,
        x: *const f32,
        n: u64,
        quants: *mut i8,
        scales: *mut f32,
        halves: *mut u16,
        fused: *mut c_int,
    ) -> cera_hip_status;
    pub fn cera_hip_attn_decode(
        ctx: *mut cera_hip_ctx,
        q: *const f32,
        k: *const f32,
        v: *const f32,
        n_heads: u32,
        n_kv_heads: u32,
        head_dim: u32,
        seq_len: u64,
        scale: f32,
        n_splits: u32,
        out: *mut f32,
    ) -> cera_hip_status;
    pub fn cera_hip_attn_prefill(
        ctx: *mut cera_hip_ctx,
        q: *const f32,
        k: *const f32,
        v: *const f32,
        n_heads: u32,
        n_kv_heads: u32,
        head_dim: u32,
        start_pos: u64,
        n_queries: u32,
        scale: f32,
        out: *mut f32,
    ) -> cera_hip_status;
    pub fn cera_hip_attn_f16kv(
        ctx: *mut cera_hip_ctx,
        q: *const f32,
        k: *const f32,
        v: *const f32,
        n_heads: u32,
        n_kv_heads: u32,
        head_dim: u32,
        start_pos: u64,
        n_queries: u32,
        scale: f32,
        n_splits: u32,
        out: *mut f32,
    ) -> cera_hip_status;
    pub fn cera_hip_rmsnorm(
        ctx: *mut cera_hip_ctx,
        x: *const f32,
        weight: *const f32,
        n: u64,
        eps: f32,
        y: *mut f32,
    ) -> cera_hip_status;
    pub fn cera_hip_silu_mul(
        ctx: *mut cera_hip_ctx,
        gate: *const f32,
        up: *const f32,
        n: u64,
        out: *mut f32,
    ) -> cera_hip_status;
    pub fn cera_hip_rope(
        ctx: *mut cera_hip_ctx,
        q: *mut f32,
        k: *mut f32,
        pos: u32,
        n_heads: u32,
        n_kv_heads: u32,
        head_dim: u32,
        freq_base: f32,
        rope_type: u32,
        freq_factors: *const f32,
    ) -> cera_hip_status;
    pub fn cera_hip_argmax(
        ctx: *mut cera_hip_ctx,
        logits: *const f32,
        n: u64,
        index: *mut u32,
    ) -> cera_hip_status;
    pub fn cera_hip_dequantize_row(
        ctx: *mut cera_hip_ctx,
        w: *const cera_hip_tensor,
        row: u64,
        out: *mut f32,
    ) -> cera_hip_status;
    pub fn cera_hip_rmsnorm_q8_0(
        ctx: *mut cera_hip_ctx,
        x: *const f32,
        weight: *const f32,
        n: u64,
        eps: f32,
        y: *mut f32,
        scales: *mut f32,
        quants: *mut i8,
    ) -> cera_hip_status;
    pub fn cera_hip_attn_decode_step(
        ctx: *mut cera_hip_ctx,
        q: *const f32,
        k_new: *const f32,
        v_new: *const f32,
        k_cache: *const f32,
        v_cache: *const f32,
        n_heads: u32,
        n_kv_heads: u32,
        head_dim: u32,
        pos: u32,
        rope_base: f32,
        rope_type: u32,
        freq_factors: *const f32,
        scale: f32,
        kv_type: u32,
        out: *mut f32,
        out_scales: *mut f32,
        out_quants: *mut i8,
        k_row: *mut f32,
        v_row: *mut f32,
    ) -> cera_hip_status;
    pub fn cera_hip_ffn_gate_up_fused(
        ctx: *mut cera_hip_ctx,
        gate: *const cera_hip_tensor,
        up: *const cera_hip_tensor,
        x: *const f32,
        norm_w: *const f32,
        eps: f32,
        quants: *mut i8,
        scales: *mut f32,
    ) -> cera_hip_status;
    pub fn cera_hip_qkv_fused(
        ctx: *mut cera_hip_ctx,
        a: *const cera_hip_tensor,
        b: *const cera_hip_tensor,
        x: *const f32,
        norm_w: *const f32,
        eps: f32,
        ya: *mut f32,
        yb: *mut f32,
    ) -> cera_hip_status;
    pub fn cera_hip_gemv_reference_order(
        ctx: *mut cera_hip_ctx,
        w: *const cera_hip_tensor,
        x: *const f32,
        y: *mut f32,
    ) -> cera_hip_status;
    pub fn cera_hip_attn_decode_reference_order(
        ctx: *mut cera_hip_ctx,
        q: *const f32,
        k: *const f32,
        v: *const f32,
        n_heads: u32,
        n_kv_heads: u32,
        head_dim: u32,
        seq_len: u64,
        scale: f32,
        out: *mut f32,
    ) -> cera_hip_status;
    pub fn cera_hip_rmsnorm_reference_order(
        ctx: *mut cera_hip_ctx,
        x: *const f32,
        weight: *const f32,
        n: u64,
        eps: f32,
        y: *mut f32,
    ) -> cera_hip_status;
    pub fn cera_hip_gemm_reference_order(
        ctx: *mut cera_hip_ctx,
        w: *const cera_hip_tensor,
        x: *const f32,
        n: u64,
        x86_repack: u32,
        out: *mut f32,
    ) -> cera_hip_status;
    pub fn cera_hip_flash_attn_reference_order(
        ctx: *mut cera_hip_ctx,
        q: *const f32,
        k: *const f32,
        v: *const f32,
        n_queries: u32,
        n_heads: u32,
        n_kv_heads: u32,
        head_dim: u32,
        start_pos: u32,
        scale: f32,
        out: *mut f32,
    ) -> cera_hip_status;
    pub fn cera_hip_quantize_q8_0_dev(
        ctx: *mut cera_hip_ctx,
        x: *const f32,
        k: u64,
        scales: *mut f32,
        quants: *mut i8,
    ) -> cera_hip_status;
    pub fn cera_hip_gemv_q8_dev(
        ctx: *mut cera_hip_ctx,
        w: *const cera_hip_dtensor,
        xs: *const f32,
        xq: *const i8,
        y: *mut f32,
    ) -> cera_hip_status;
    pub fn cera_hip_gemv_seq_dev(
        ctx: *mut cera_hip_ctx,
        ops: *const cera_hip_gemv_op,
        n: u32,
    ) -> cera_hip_status;
    pub fn cera_hip_decode_ops_dev(
        ctx: *mut cera_hip_ctx,
        ops: *const cera_hip_decode_op,
        n: u32,
    ) -> cera_hip_status;
    pub fn cera_hip_attn_decode_dev(
        ctx: *mut cera_hip_ctx,
        q: *const f32,
        k_headmajor: *const f32,
        v_headmajor: *const f32,
        n_heads: u32,
        n_kv_heads: u32,
        head_dim: u32,
        seq_len: u64,
        max_seq: u64,
        scale: f32,
        n_splits: u32,
        out: *mut f32,
    ) -> cera_hip_status;
    pub fn cera_hip_attn_decode_dev_noalloc(
        ctx: *mut cera_hip_ctx,
        q: *const f32,
        k_headmajor: *const f32,
        v_headmajor: *const f32,
        n_heads: u32,
        n_kv_heads: u32,
        head_dim: u32,
        seq_len: u64,
        max_seq: u64,
        scale: f32,
        n_splits: u32,
        out: *mut f32,
    ) -> cera_hip_status;
    pub fn cera_hip_attn_decode_f16_dev(
        ctx: *mut cera_hip_ctx,
        q: *const f32,
        k_headmajor_f16: *const c_void,
        v_headmajor_f16: *const c_void,
        n_heads: u32,
        n_kv_heads: u32,
        head_dim: u32,
        seq_len: u64,
        max_seq: u64,
        scale: f32,
        n_splits: u32,
        out: *mut f32,
    ) -> cera_hip_status;
    pub fn cera_hip_gemm_dev(
        ctx: *mut cera_hip_ctx,
        w: *const cera_hip_dtensor,
        x: *const f32,
        n: u64,
        out: *mut f32,
    ) -> cera_hip_status;
    pub fn cera_hip_model_create(
        ctx: *mut cera_hip_ctx,
        config: *const cera_hip_config,
        token_embd: *const cera_hip_tensor,
        output: *const cera_hip_tensor,
        output_norm: *const f32,
        layers: *const cera_hip_layer,
        out: *mut *mut cera_hip_model,
    ) -> cera_hip_status;
    pub fn cera_hip_model_destroy(model: *mut cera_hip_model);
    pub fn cera_hip_forward(
        model: *mut cera_hip_model,
        token: u32,
        pos: u32,
        logits: *mut f32,
    ) -> cera_hip_status;
    pub fn cera_hip_forward_greedy(
        model: *mut cera_hip_model,
        token: u32,
        pos: u32,
        next: *mut u32,
    ) -> cera_hip_status;
    pub fn cera_hip_forward_prefill(
        model: *mut cera_hip_model,
        tokens: *const u32,
        n: u32,
        start_pos: u32,
        last_logits: *mut f32,
    ) -> cera_hip_status;
    pub fn cera_hip_forward_prefill_logits_all(
        model: *mut cera_hip_model,
        tokens: *const u32,
        n: u32,
        start_pos: u32,
        logits_all: *mut f32,
    ) -> cera_hip_status;
    pub fn cera_hip_configure_kv(model: *mut cera_hip_model, kv_type: u32) -> cera_hip_status;
    pub fn cera_hip_kv_type(model: *const cera_hip_model) -> u32;
    pub fn cera_hip_set_reference_order(model: *mut cera_hip_model, on: u32) -> cera_hip_status;
    pub fn cera_hip_reference_order(model: *const cera_hip_model) -> u32;
    pub fn cera_hip_truncate_kv(model: *mut cera_hip_model, len: u32) -> cera_hip_status;
    pub fn cera_hip_seq_len(model: *const cera_hip_model) -> u32;
    pub fn cera_hip_memory_bytes(model: *const cera_hip_model) -> u64;
    pub fn cera_hip_drop_decode_copies(model: *mut cera_hip_model, freed_bytes: *mut u64) -> cera_hip_status;
    pub fn cera_hip_shift_kv(
        model: *mut cera_hip_model,
        n_keep: u32,
        shift: u32,
    ) -> cera_hip_status;
    pub fn cera_hip_read_kv(
        model: *mut cera_hip_model,
        layer: u32,
        k_out: *mut f32,
        v_out: *mut f32,
    ) -> cera_hip_status;
    pub fn cera_hip_write_kv(
        model: *mut cera_hip_model,
        layer: u32,
        k: *const f32,
        v: *const f32,
        n_pos: u32,
    ) -> cera_hip_status;
    pub fn cera_hip_set_seq_len(model: *mut cera_hip_model, len: u32) -> cera_hip_status;
    pub fn cera_hip_read_hidden(
        model: *mut cera_hip_model,
        hidden_out: *mut f32,
    ) -> cera_hip_status;
}

#[cfg(test)]
mod tests {
    use super::*;
    use std::mem::{align_of, size_of};

    /// The layouts the C header fixes on LP64.
    #[test]
    fn struct_layouts_match_the_header() {
        assert_eq!(size_of::<cera_hip_tensor>(), 40);
        assert_eq!(size_of::<cera_hip_layer>(), 2 * 8 + 7 * 40 + 5 * 8);
        assert_eq!(size_of::<cera_hip_config>(), 9 * 4 + 6 * 4 + 4 + 8);
        assert_eq!(align_of::<cera_hip_config>(), 8);
        assert_eq!(size_of::<cera_hip_gemv_op>(), 40);
        assert_eq!(size_of::<cera_hip_decode_op>(), 104);
    }
}
