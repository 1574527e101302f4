//! Dense llama-family transformers (LLaMA / Mistral / Qwen2 / Qwen3 / Granite) on an AMD
//! MI355X through `libcera_hip.so` (crate `cera-hip-sys`).
//!
//! The library owns everything device-side: the weights in their native GGUF block layout in
//! HBM, the KV cache, the position counter and the whole per-token launch graph. This type is
//! the thin `Model` face over it, shaped like the other device-resident backends
//! (`GpuLfm2Model`, `MetalLfm2Model`): the CPU-side [`InferenceState`] only mirrors `seq_len`.
//!
//! Weights come from the same [`GpuWeightSource`] the wgpu and Metal loaders consume, so GGUF
//! parsing, dtype resolution and the optional-tensor rules (QK-norm, QKV bias, untied head,
//! Llama-3 `rope_freqs`, Granite scalars) are not restated here.
//!
//! Threading: the library serialises every call on a model behind the model's own mutex and
//! every call on a context behind the context's, which is the role `infer_lock` plays in the
//! other GPU backends; the raw pointers below are therefore safe to share.

use std::ffi::CStr;
use std::sync::OnceLock;

use anyhow::{Context, Result, bail};
use cera_hip_sys as sys;

use crate::CeraError;
use crate::backend::cpu::RopeType;
use crate::kv_cache::{InferenceState, KvCompression, LayerSnapshot, StateSnapshot};
use crate::model::gpu_weight_source::GpuWeightSource;
use crate::model::transformer::{self, WeightRef};
use crate::model::{Model, ModelConfig};
use crate::tensor::DType;

/// KV cache element type, as configured by the first session (`configure_kv_compression`).
#[derive(Debug, Clone, Copy, PartialEq, Eq)]
enum KvMode {
    F32,
    F16,
}

impl KvMode {
    fn label(self) -> &'static str {
        match self {
            KvMode::F32 => "none",
            KvMode::F16 => "f16",
        }
    }
    fn id(self) -> u32 {
        match self {
            KvMode::F32 => sys::CERA_HIP_KV_F32,
            KvMode::F16 => sys::CERA_HIP_KV_F16,
        }
    }
}

pub struct HipLlamaModel {
    ctx: *mut sys::cera_hip_ctx,
    model: *mut sys::cera_hip_model,
    config: ModelConfig,
    /// First `configure_kv_compression` wins; later calls must agree.
    kv_mode: OnceLock<KvMode>,
}

// SAFETY: `ctx` and `model` are only ever passed to `libcera_hip.so`, which takes the model's
// lock (and the context's) around every entry point; no Rust-side state is mutated through
// `&self` except the `OnceLock`.
unsafe impl Send for HipLlamaModel {}
unsafe impl Sync for HipLlamaModel {}

/// GGML type id of a cera dtype, as `cera_hip_tensor::ggml_type` wants it.
fn ggml_type_id(dtype: DType) -> Result<u32> {
    Ok(match dtype {
        DType::F32 => sys::CERA_HIP_F32,
        DType::F16 => sys::CERA_HIP_F16,
        DType::BF16 => sys::CERA_HIP_BF16,
        DType::Q4_0 => sys::CERA_HIP_Q4_0,
        DType::Q4_1 => sys::CERA_HIP_Q4_1,
        DType::Q8_0 => sys::CERA_HIP_Q8_0,
        DType::Q4KM => sys::CERA_HIP_Q4_K,
        DType::Q5KM => sys::CERA_HIP_Q5_K,
        DType::Q6K => sys::CERA_HIP_Q6_K,
        other => bail!("dtype {other:?} has no GGML id the hip backend accepts"),
    })
}

/// Describe one weight matrix to the library: shape, type and the mmap slice that holds it. The
/// slice is only borrowed until `cera_hip_model_create` returns.
fn tensor_of(src: &dyn GpuWeightSource, wref: &WeightRef) -> Result<sys::cera_hip_tensor> {
    let bytes = src.weight_bytes(wref);
    Ok(sys::cera_hip_tensor {
        ggml_type: ggml_type_id(wref.dtype)?,
        _reserved: 0,
        m: wref.m as u64,
        k: wref.k as u64,
        data: bytes.as_ptr().cast(),
        nbytes: bytes.len() as u64,
    })
}

fn opt_ptr(v: Option<&[f32]>) -> *const f32 {
    v.map_or(std::ptr::null(), |s| s.as_ptr())
}

/// Message of the last failure on `ctx` (or the process-wide one when `ctx` is null).
fn last_error(ctx: *const sys::cera_hip_ctx) -> String {
    // SAFETY: the library returns a NUL-terminated string that stays valid until the next call
    // on the same context; it is copied out immediately.
    unsafe {
        let p = sys::cera_hip_last_error(ctx);
        if p.is_null() {
            String::from("unknown error")
        } else {
            CStr::from_ptr(p).to_string_lossy().into_owned()
        }
    }
}

fn status_name(st: sys::cera_hip_status) -> &'static str {
    match st {
        sys::CERA_HIP_OK => "ok",
        sys::CERA_HIP_ERR_DEVICE => "device error",
        sys::CERA_HIP_ERR_OOM => "out of memory",
        sys::CERA_HIP_ERR_UNSUPPORTED_DTYPE => "unsupported dtype",
        sys::CERA_HIP_ERR_SHAPE => "unsupported shape",
        sys::CERA_HIP_ERR_POSITION => "position mismatch",
        sys::CERA_HIP_ERR_ARGUMENT => "bad argument",
        _ => "unknown status",
    }
}

impl HipLlamaModel {
    /// Upload a dense transformer described by `src` to HIP device 0.
    ///
    /// `CERA_HIP_HSACO`, when set, names the standalone gfx950 code object to launch the
    /// quantizer and GEMV kernels from (`hipModuleLoad`); unset, the kernels embedded in the
    /// library are used.
    pub(crate) fn from_weight_source(
        src: &dyn GpuWeightSource,
        context_size: usize,
    ) -> Result<Self> {
        let mut config = src.config().clone();
        // Clamp the context like the other GPU loaders do, so the engine sees the effective limit.
        config.max_seq_len = context_size.min(config.max_seq_len);
        anyhow::ensure!(
            config.moe.is_none(),
            "the hip backend serves dense transformers only (no mixture-of-experts layers)"
        );
        let n_kv_heads = config.n_kv_heads;
        anyhow::ensure!(
            config.kv_heads_per_layer.iter().all(|&h| h == n_kv_heads),
            "the hip backend needs the same KV head count in every layer"
        );

        let embd = transformer::resolve_weight(src.gguf(), "token_embd.weight")?;
        let embd_t = tensor_of(src, &embd).context("token_embd.weight")?;
        let output_t = match src.output_ref() {
            Some(w) => Some(tensor_of(src, w).context("output.weight")?),
            None => None,
        };

        let mut layers = Vec::with_capacity(config.n_layers);
        for l in 0..config.n_layers {
            let need = |w: Option<&WeightRef>, what: &str| -> Result<sys::cera_hip_tensor> {
                let w = w.with_context(|| format!("layer {l}: missing {what}"))?;
                tensor_of(src, w).with_context(|| format!("layer {l}: {what}"))
            };
            layers.push(sys::cera_hip_layer {
                attn_norm: src.attn_norm_weight(l).as_ptr(),
                ffn_norm: src.ffn_norm_weight(l).as_ptr(),
                attn_q: need(src.attn_q_ref(l), "attn_q")?,
                attn_k: need(src.attn_k_ref(l), "attn_k")?,
                attn_v: need(src.attn_v_ref(l), "attn_v")?,
                attn_output: need(src.attn_output_ref(l), "attn_output")?,
                ffn_gate: need(Some(src.ffn_gate_ref(l)?), "ffn_gate")?,
                ffn_up: need(Some(src.ffn_up_ref(l)?), "ffn_up")?,
                ffn_down: need(Some(src.ffn_down_ref(l)?), "ffn_down")?,
                q_bias: opt_ptr(src.attn_q_bias(l)),
                k_bias: opt_ptr(src.attn_k_bias(l)),
                v_bias: opt_ptr(src.attn_v_bias(l)),
                q_norm: opt_ptr(src.attn_q_norm_weight(l)),
                k_norm: opt_ptr(src.attn_k_norm_weight(l)),
            });
        }

        let u32_of = |v: usize, what: &str| -> Result<u32> {
            u32::try_from(v).with_context(|| format!("{what} = {v} does not fit 32 bits"))
        };
        let cfg = sys::cera_hip_config {
            n_layers: u32_of(config.n_layers, "n_layers")?,
            hidden: u32_of(config.hidden_size, "hidden_size")?,
            ffn: u32_of(config.intermediate_size, "intermediate_size")?,
            n_heads: u32_of(config.n_heads, "n_heads")?,
            n_kv_heads: u32_of(config.n_kv_heads, "n_kv_heads")?,
            head_dim: u32_of(config.head_dim, "head_dim")?,
            vocab: u32_of(config.vocab_size, "vocab_size")?,
            max_seq_len: u32_of(config.max_seq_len, "max_seq_len")?,
            rope_type: match src.rope_type() {
                RopeType::Neox => 0,
                RopeType::Norm => 1,
            },
            rope_theta: config.rope_theta,
            rms_eps: config.rms_norm_eps,
            embed_scale: config.scalars.embedding,
            residual_scale: config.scalars.residual,
            // 0 selects the default 1/sqrt(head_dim); Granite's multiplier replaces it.
            attn_scale: config.scalars.attn.unwrap_or(0.0),
            logit_scale: config.scalars.logit,
            rope_freqs: opt_ptr(src.rope_freqs()),
        };

        let hsaco = std::env::var_os("CERA_HIP_HSACO")
            .map(|p| {
                std::ffi::CString::new(p.to_string_lossy().into_owned())
                    .context("CERA_HIP_HSACO contains a NUL byte")
            })
            .transpose()?;
        let hsaco_ptr = hsaco.as_ref().map_or(std::ptr::null(), |c| c.as_ptr());

        let mut ctx: *mut sys::cera_hip_ctx = std::ptr::null_mut();
        // SAFETY: plain FFI call; `ctx` receives an owned handle on success.
        let st = unsafe { sys::cera_hip_ctx_create(0, hsaco_ptr, &mut ctx) };
        if st != sys::CERA_HIP_OK {
            bail!(
                "hip context: {} ({})",
                last_error(std::ptr::null()),
                status_name(st)
            );
        }

        let mut model: *mut sys::cera_hip_model = std::ptr::null_mut();
        // SAFETY: every pointer handed over (config, tensors, norm vectors, the mmap slices the
        // tensors point into) outlives this call, which is all the library asks for: it copies
        // the weights to device memory before returning.
        let st = unsafe {
            sys::cera_hip_model_create(
                ctx,
                &cfg,
                &embd_t,
                output_t.as_ref().map_or(std::ptr::null(), |t| t as *const _),
                src.output_norm_weight().as_ptr(),
                layers.as_ptr(),
                &mut model,
            )
        };
        if st != sys::CERA_HIP_OK {
            let msg = last_error(ctx);
            // SAFETY: `ctx` came from cera_hip_ctx_create above and is not used afterwards.
            unsafe { sys::cera_hip_ctx_destroy(ctx) };
            bail!("hip model upload: {msg} ({})", status_name(st));
        }

        // SAFETY: `model` is a live handle.
        let bytes = unsafe { sys::cera_hip_memory_bytes(model) };
        tracing::info!(
            "HIP model: {} layers, hs={}, is={}, vocab={}, {:.2} GB in HBM",
            config.n_layers,
            config.hidden_size,
            config.intermediate_size,
            config.vocab_size,
            bytes as f64 / 1e9
        );

        Ok(Self {
            ctx,
            model,
            config,
            kv_mode: OnceLock::new(),
        })
    }

    /// Panic with the library's message when a forward-path call failed. The forward methods of
    /// `Model` are infallible by signature; the other GPU backends `expect()` here as well. What
    /// can reach this are caller bugs (position mismatch, out-of-range token) and device loss.
    fn expect_ok(&self, st: sys::cera_hip_status, what: &str) {
        if st != sys::CERA_HIP_OK {
            panic!(
                "hip backend: {what} failed: {} ({})",
                last_error(self.ctx),
                status_name(st)
            );
        }
    }

    fn device_seq_len(&self) -> usize {
        // SAFETY: `model` is a live handle.
        unsafe { sys::cera_hip_seq_len(self.model) as usize }
    }

    fn kv_is_f16(&self) -> bool {
        // SAFETY: `model` is a live handle.
        unsafe { sys::cera_hip_kv_type(self.model) == sys::CERA_HIP_KV_F16 }
    }

    fn pos_u32(pos: usize) -> u32 {
        u32::try_from(pos).expect("position exceeds 32 bits")
    }
}

impl Drop for HipLlamaModel {
    fn drop(&mut self) {
        // SAFETY: both handles are owned by `self` and not used after this.
        unsafe {
            sys::cera_hip_model_destroy(self.model);
            sys::cera_hip_ctx_destroy(self.ctx);
        }
    }
}

impl Model for HipLlamaModel {
    fn forward(&self, tokens: &[u32], pos: usize, state: &mut InferenceState) -> Vec<f32> {
        assert_eq!(tokens.len(), 1, "forward takes exactly one token");
        let mut logits = vec![0f32; self.config.vocab_size];
        // `pos == 0` starts a fresh sequence on the device (a new `InferenceState` per
        // `generate()`), otherwise `pos` must equal the device's sequence length.
        // SAFETY: `logits` holds `vocab` floats, which is what the call writes.
        let st = unsafe {
            sys::cera_hip_forward(
                self.model,
                tokens[0],
                Self::pos_u32(pos),
                logits.as_mut_ptr(),
            )
        };
        self.expect_ok(st, "forward");
        state.seq_len = self.device_seq_len();
        logits
    }

    fn forward_greedy(&self, tokens: &[u32], pos: usize, state: &mut InferenceState) -> u32 {
        assert_eq!(tokens.len(), 1, "forward_greedy takes exactly one token");
        let mut next = 0u32;
        // The arg-max runs on the device: four bytes come back instead of `vocab` floats.
        // SAFETY: `next` is a valid `u32` slot.
        let st = unsafe {
            sys::cera_hip_forward_greedy(self.model, tokens[0], Self::pos_u32(pos), &mut next)
        };
        self.expect_ok(st, "forward_greedy");
        state.seq_len = self.device_seq_len();
        next
    }

    fn forward_prefill(
        &self,
        tokens: &[u32],
        start_pos: usize,
        state: &mut InferenceState,
    ) -> Vec<f32> {
        if tokens.is_empty() {
            return Vec::new();
        }
        let mut logits = vec![0f32; self.config.vocab_size];
        let n = u32::try_from(tokens.len()).expect("prompt longer than 2^32 tokens");
        // SAFETY: `tokens` holds `n` ids; `logits` holds `vocab` floats.
        let st = unsafe {
            sys::cera_hip_forward_prefill(
                self.model,
                tokens.as_ptr(),
                n,
                Self::pos_u32(start_pos),
                logits.as_mut_ptr(),
            )
        };
        self.expect_ok(st, "forward_prefill");
        state.seq_len = self.device_seq_len();
        logits
    }

    fn supports_all_logits(&self) -> bool {
        true
    }

    fn forward_prefill_logits_all(
        &self,
        tokens: &[u32],
        start_pos: usize,
        state: &mut InferenceState,
    ) -> Vec<f32> {
        if tokens.is_empty() {
            return Vec::new();
        }
        let mut all = vec![0f32; tokens.len() * self.config.vocab_size];
        let n = u32::try_from(tokens.len()).expect("batch longer than 2^32 tokens");
        // SAFETY: `all` holds `n * vocab` floats, row-major, which is what the call writes.
        let st = unsafe {
            sys::cera_hip_forward_prefill_logits_all(
                self.model,
                tokens.as_ptr(),
                n,
                Self::pos_u32(start_pos),
                all.as_mut_ptr(),
            )
        };
        self.expect_ok(st, "forward_prefill_logits_all");
        state.seq_len = self.device_seq_len();
        all
    }

    /// The KV cache and its length live on the device: rewind both, then the mirror.
    fn truncate_kv(&self, state: &mut InferenceState, len: usize) {
        assert!(
            len <= state.seq_len,
            "truncate_kv({len}) exceeds seq_len {}",
            state.seq_len
        );
        if len != self.device_seq_len() {
            // SAFETY: `model` is a live handle.
            let st = unsafe { sys::cera_hip_truncate_kv(self.model, Self::pos_u32(len)) };
            self.expect_ok(st, "truncate_kv");
        }
        state.seq_len = len;
    }

    fn config(&self) -> &ModelConfig {
        &self.config
    }

    fn supports_kv_shift(&self) -> bool {
        // the shift kernel is instantiated for the head sizes models use
        matches!(self.config.head_dim, 32 | 64 | 80 | 96 | 128 | 256)
    }

    fn shift_kv(&self, state: &mut InferenceState, n_keep: usize, shift: usize) {
        assert!(shift > 0, "shift_kv: shift must be positive");
        assert!(
            n_keep + shift <= state.seq_len,
            "shift_kv: n_keep + shift exceeds seq_len"
        );
        // Drops cells [n_keep, n_keep + shift), moves the tail down and re-rotates its K rows on
        // the device.
        // SAFETY: `model` is a live handle.
        let st = unsafe {
            sys::cera_hip_shift_kv(self.model, Self::pos_u32(n_keep), Self::pos_u32(shift))
        };
        self.expect_ok(st, "shift_kv");
        state.seq_len = self.device_seq_len();
    }

    fn gpu_memory_bytes(&self) -> u64 {
        // SAFETY: `model` is a live handle.
        unsafe { sys::cera_hip_memory_bytes(self.model) }
    }

    fn f16_kv_supported(&self) -> bool {
        true
    }

    fn configure_kv_compression(&self, compression: &KvCompression) -> Result<(), CeraError> {
        let want = match compression {
            KvCompression::None => KvMode::F32,
            KvCompression::F16 => KvMode::F16,
            KvCompression::TurboQuant { .. } => {
                // Not an error: like a TurboQuant request another backend cannot serve, stay on
                // the uncompressed cache and say so.
                tracing::warn!(
                    target: "cera::hip",
                    "TurboQuant requested but not available on the hip backend; \
                     falling back to f32 KV"
                );
                KvMode::F32
            }
        };
        if let Some(&configured) = self.kv_mode.get() {
            if configured != want {
                return Err(CeraError::KvCompressionConflict {
                    configured: configured.label().to_string(),
                    requested: want.label().to_string(),
                });
            }
            return Ok(()); // same mode again: the `Session::reset` path
        }
        // SAFETY: `model` is a live handle.
        let st = unsafe { sys::cera_hip_configure_kv(self.model, want.id()) };
        if st != sys::CERA_HIP_OK {
            // Another thread configured a different mode first, or the cache is not empty.
            let current = if self.kv_is_f16() {
                KvMode::F16
            } else {
                KvMode::F32
            };
            if current != want {
                return Err(CeraError::KvCompressionConflict {
                    configured: current.label().to_string(),
                    requested: want.label().to_string(),
                });
            }
            return Err(CeraError::Backend(format!(
                "hip: configure_kv failed: {}",
                last_error(self.ctx)
            )));
        }
        let _ = self.kv_mode.set(want);
        Ok(())
    }

    /// Prefix-cache snapshot: per layer, cache rows `[0, seq_len)` in the reference's time-major
    /// `[pos][kv_dim]` order. The library hands rows out as f32 whatever the cache holds; an f16
    /// cache widens exactly, so narrowing back to half here is lossless and yields the same
    /// `AttentionF16` bytes a CPU f16 state would snapshot.
    fn snapshot_state(&self) -> StateSnapshot {
        let seq_len = self.device_seq_len();
        let kv_dim = self.config.n_kv_heads * self.config.head_dim;
        let f16 = self.kv_is_f16();
        let mut layers = Vec::with_capacity(self.config.n_layers);
        let mut k = vec![0f32; seq_len * kv_dim];
        let mut v = vec![0f32; seq_len * kv_dim];
        for l in 0..self.config.n_layers {
            if seq_len > 0 {
                // SAFETY: both buffers hold `seq_len * kv_dim` floats, which is what is written.
                let st = unsafe {
                    sys::cera_hip_read_kv(self.model, l as u32, k.as_mut_ptr(), v.as_mut_ptr())
                };
                self.expect_ok(st, "snapshot_state");
            }
            let pack = |x: &[f32]| -> Vec<u8> {
                if f16 {
                    x.iter()
                        .flat_map(|&f| half::f16::from_f32(f).to_bits().to_le_bytes())
                        .collect()
                } else {
                    x.iter().flat_map(|f| f.to_le_bytes()).collect()
                }
            };
            let (k_data, v_data) = (pack(&k), pack(&v));
            layers.push(if f16 {
                LayerSnapshot::AttentionF16 { k_data, v_data }
            } else {
                LayerSnapshot::Attention { k_data, v_data }
            });
        }
        StateSnapshot { layers, seq_len }
    }

    fn restore_state(&self, snapshot: &StateSnapshot) {
        assert_eq!(
            snapshot.layers.len(),
            self.config.n_layers,
            "snapshot has a different layer count"
        );
        let kv_dim = self.config.n_kv_heads * self.config.head_dim;
        let n = snapshot.seq_len;
        let f16 = self.kv_is_f16();
        for (l, layer) in snapshot.layers.iter().enumerate() {
            let (k_bytes, v_bytes, half_wide) = match layer {
                LayerSnapshot::Attention { k_data, v_data } => (k_data, v_data, false),
                LayerSnapshot::AttentionF16 { k_data, v_data } => (k_data, v_data, true),
                _ => panic!("hip backend: snapshot layer {l} is not a plain attention layer"),
            };
            assert_eq!(
                half_wide, f16,
                "snapshot element width does not match the configured KV cache"
            );
            let unpack = |b: &[u8]| -> Vec<f32> {
                if half_wide {
                    b.chunks_exact(2)
                        .map(|c| half::f16::from_bits(u16::from_le_bytes([c[0], c[1]])).to_f32())
                        .collect()
                } else {
                    b.chunks_exact(4)
                        .map(|c| f32::from_le_bytes([c[0], c[1], c[2], c[3]]))
                        .collect()
                }
            };
            let (k, v) = (unpack(k_bytes), unpack(v_bytes));
            assert!(
                k.len() >= n * kv_dim && v.len() >= n * kv_dim,
                "snapshot layer {l} is shorter than its seq_len"
            );
            if n > 0 {
                // SAFETY: both slices hold at least `n * kv_dim` floats, which is what is read.
                let st = unsafe {
                    sys::cera_hip_write_kv(
                        self.model,
                        l as u32,
                        k.as_ptr(),
                        v.as_ptr(),
                        Self::pos_u32(n),
                    )
                };
                self.expect_ok(st, "restore_state");
            }
        }
        // SAFETY: `model` is a live handle.
        let st = unsafe { sys::cera_hip_set_seq_len(self.model, Self::pos_u32(n)) };
        self.expect_ok(st, "restore_state");
    }

    // Kept at their defaults on purpose:
    // * `forward_prefill_chunked`: the trait default already splits at `ubatch`, calls
    //   `forward_prefill` per chunk and polls `cancel` in between;
    // * `supports_embedding_input`, `supports_hidden_states`, `turboquant_supported`,
    //   `supports_moe_lora`: `false` — the library has no such entry points;
    // * `configure_cache`: no-op — the prefix cache is driven through snapshot/restore above.
}
