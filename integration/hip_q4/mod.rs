//! HIP backend of the Q4 matmul path for `crates/inference`: the wrappers the Metal backend's callers
//! already use, over `liblattice_hip_q4.so`.  Meant to live at
//! `crates/inference/src/forward/hip_q4/mod.rs`, compiled under `#[cfg(feature = "hip-gpu")]` beside
//! the `#[cfg(all(target_os = "macos", feature = "metal-gpu"))]` arm of `forward/metal_qwen35.rs`.
//!
//! What each item replaces (reference file:line):
//!   `HipQ4WeightBuf`            `Q4WeightBuf`                          metal_qwen35.rs:599-636
//!   `mmap_q4_weight`            `mmap_q4_weight`                       metal_qwen35.rs:660-702
//!   `dispatch_matmul`           `dispatch_matmul` / `_q4`              inner/dispatch.rs:231, 148-168
//!   `dispatch_gemm`             `dispatch_gemm`                        inner/dispatch.rs:507-525
//!   `dispatch_gemm_at`          `dispatch_gemm_at`                     inner/dispatch.rs:935-960
//!   `dispatch_lora_if_active`   `dispatch_lora_if_active`              inner/layers/mod.rs:15-51
//!   `load_lora_adapter`         `load_lora_adapter`                    metal_qwen35.rs:3806-3986
//!   `encode_token_chain`        the dispatches `forward_step` encodes  metal_qwen35.rs:6943, 6447
//!
//! Conventions kept from the Metal backend: byte offsets into buffers, `n == 0` / `m == 0` are silent
//! no-ops, `k % 32 != 0` is a programming error (assert), every output element is overwritten, loaders
//! return `Result<_, String>`.  A Metal `Buffer` becomes a `DevBuf` (device pointer + length); the
//! command encoder becomes a HIP stream.
//!
//! Not compiled here (the build image has no `rustc`).

pub mod ffi;

use ffi::*;
use std::collections::HashMap;
use std::os::raw::c_void;
use std::ptr;

/// A device allocation handed to the dispatch functions (the role `metal::Buffer` plays today).
pub struct DevBuf {
    pub ptr: *mut c_void,
    pub len: usize,
}

impl DevBuf {
    fn at(&self, byte_offset: u64) -> *mut c_void {
        assert!(byte_offset as usize <= self.len, "offset {byte_offset} past a {}-byte buffer", self.len);
        // SAFETY: in bounds of the allocation by the assert above.
        unsafe { (self.ptr as *mut u8).add(byte_offset as usize) as *mut c_void }
    }
}

/// Resident Q4 tensor: the file's bytes copied verbatim to HBM, payload addressed by offset.
pub struct HipQ4WeightBuf {
    raw: *mut Lq4Weight,
    /// Bytes from the start of the buffer to the first block (the `.q4` header length).
    pub payload_offset: u64,
}

impl Drop for HipQ4WeightBuf {
    fn drop(&mut self) {
        // SAFETY: raw came from lq4_weight_upload and is freed exactly once.
        unsafe { lq4_weight_free(self.raw) };
    }
}

/// One MoE layer's resident tensors (the role of `MoeMetalBuffers`, metal_qwen35.rs): expert-major
/// `gate_up [E, 2*inter, hidden]` and `down [E, hidden, inter]`, the shared expert's fused
/// `shared_gate_up [2*shared_inter, hidden]` (gate_proj rows, then up_proj rows) and
/// `shared_down [hidden, shared_inter]`, and its f32 gate vector `[hidden]`.
pub struct HipMoeLayer {
    pub gate_up: HipQ4WeightBuf,
    pub down: HipQ4WeightBuf,
    pub shared_gate_up: HipQ4WeightBuf,
    pub shared_down: HipQ4WeightBuf,
    pub shared_expert_gate: DevBuf,
    pub num_experts: u32,
    pub top_k: u32,
    pub inter: u32,
    pub shared_inter: u32,
    pub hidden: u32,
}

struct HipLoraProjection {
    raw: *mut Lq4Lora,
}

impl Drop for HipLoraProjection {
    fn drop(&mut self) {
        // SAFETY: raw came from lq4_lora_upload and is freed exactly once.
        unsafe { lq4_lora_free(self.raw) };
    }
}

/// Same fields as the reference's `LoraLayerData` (metal_qwen35.rs:1701-1716).
pub struct LoraLayerData {
    pub layer_idx: usize,
    pub module: String,
    pub a: Vec<f32>, // [rank, d_in] row-major
    pub b: Vec<f32>, // [d_out, rank] row-major
    pub rank: usize,
    pub d_in: usize,
    pub d_out: usize,
}

struct HipLoraAdapter {
    projections: Vec<HashMap<String, HipLoraProjection>>,
    scale: f32,
}

/// One GPU's Q4 backend: context, stream, the model's configuration, optional adapter.
pub struct HipQ4Backend {
    ctx: *mut Lq4Ctx,
    stream: *mut c_void, // hipStream_t; null = the default stream
    config: crate::model::qwen35_config::Qwen35Config,
    lora: Option<HipLoraAdapter>,
}

impl Drop for HipQ4Backend {
    fn drop(&mut self) {
        self.lora = None; // projections before the context
        // SAFETY: ctx came from lq4_ctx_create.
        unsafe { lq4_ctx_destroy(self.ctx) };
    }
}

impl HipQ4Backend {
    /// `config`: the engine's model configuration, as the Metal state reads it from `self.engine.config`
    /// (layer count, hidden size and projection shapes for the adapter checks below).
    pub fn new(device_ordinal: i32, config: crate::model::qwen35_config::Qwen35Config) -> Result<Self, String> {
        let mut ctx = ptr::null_mut();
        // SAFETY: out pointer is valid for the call.
        check(unsafe { lq4_ctx_create(device_ordinal, &mut ctx) })?;
        Ok(Self { ctx, stream: ptr::null_mut(), config, lora: None })
    }

    /// `expected_lora_shape` (metal_qwen35.rs:3746-3768) without the Metal-only capability filter: the GDN
    /// gate projections are consumed inside a fused recurrence kernel there and rejected; this path has no such
    /// kernel, but the forward loop that would apply them is the host crate's, so the same modules are refused.
    fn expected_lora_shape(&self, layer_idx: usize, module: &str) -> Result<(usize, usize), String> {
        if matches!(module, "in_proj_b" | "in_proj_a") {
            if self.config.is_full_attention(layer_idx) {
                return Err(format!("unknown LoRA module '{module}'"));
            }
            return Err(format!(
                "module '{module}' is not yet supported in the HIP forward (consumed inside the GDN recurrence); \
                 target other GDN modules instead"
            ));
        }
        let shape = crate::lora_hook::qwen35_projection_shape(&self.config, layer_idx, module)?;
        Ok((shape.d_in, shape.d_out))
    }

    /// `mmap_q4_weight` (metal_qwen35.rs:660-702): header + shape check as today
    /// (`open_and_mmap_q4_file` with `Q4BlockCheck::Now`), then the whole file to HBM.  The ingress
    /// rule runs again inside the library (`validate = 1`); a bad block never reaches the GPU and the
    /// error names its index like `validate_q4_block_metadata_scan`.
    pub fn mmap_q4_weight(
        &self,
        path: &std::path::Path,
        _label: &str,
        expected_shape: &[usize],
    ) -> Result<HipQ4WeightBuf, String> {
        use crate::weights::q4_weights::{open_and_mmap_q4_file, Q4BlockCheck};
        let tensor_name = path.file_name().and_then(std::ffi::OsStr::to_str).unwrap_or("native Q4 tensor");
        let (header, mmap, _checked) =
            open_and_mmap_q4_file(path, Some(expected_shape), Q4BlockCheck::Now { tensor_name })?;
        let mut raw = ptr::null_mut();
        // SAFETY: mmap covers mmap.len() readable bytes for the duration of the call (the library copies).
        check(unsafe {
            lq4_weight_upload(self.ctx, mmap.as_ptr(), mmap.len(), header.payload_offset as u64, 1, &mut raw)
        })
        .map_err(|e| format!("{}: {e}", path.display()))?;
        Ok(HipQ4WeightBuf { raw, payload_offset: header.payload_offset as u64 })
    }

    /// `dispatch_matmul` (inner/dispatch.rs:231; the Q4 arm is `dispatch_matmul_q4`, :148-168):
    /// `y[n] = W[n, k] . x[k]` for one token (`m` rows up to 16 go through the same entry point).
    pub fn dispatch_matmul(&self, x: &DevBuf, qw: &HipQ4WeightBuf, y: &DevBuf, m: u32, n: u32, k: u32) {
        assert!(k > 0 && k % 32 == 0, "dispatch_matmul_q4 requires k % 32 == 0, got {k}");
        if n == 0 || m == 0 {
            return;
        }
        // SAFETY: device pointers of live allocations; the library checks shapes against the weight view.
        let rc = unsafe {
            lq4_gemv(self.ctx, qw.raw, 0, n, k, x.ptr as *const f32, m, y.ptr as *mut f32, ptr::null(), 0.0, self.stream)
        };
        check(rc).expect("lq4_gemv");
    }

    /// `dispatch_gemm` (inner/dispatch.rs:507-525): `Y[m, n] = X[m, k] . W^T`, byte offsets into x and y.
    #[allow(clippy::too_many_arguments)]
    pub fn dispatch_gemm(
        &self,
        x: &DevBuf,
        x_offset: u64,
        qw: &HipQ4WeightBuf,
        y: &DevBuf,
        y_offset: u64,
        m: u32,
        n: u32,
        k: u32,
    ) {
        self.dispatch_gemm_at(x, x_offset, qw, 0, y, y_offset, m, n, k)
    }

    /// `dispatch_gemm_at` (inner/dispatch.rs:935-960): the same over a sub-view of the weight buffer
    /// (`qw_extra_offset` bytes past the payload: fused gate||up halves, qkv||z, expert slices).
    #[allow(clippy::too_many_arguments)]
    pub fn dispatch_gemm_at(
        &self,
        x: &DevBuf,
        x_offset: u64,
        qw: &HipQ4WeightBuf,
        qw_extra_offset: u64,
        y: &DevBuf,
        y_offset: u64,
        m: u32,
        n: u32,
        k: u32,
    ) {
        assert!(k > 0 && k % 32 == 0, "dispatch_gemm_q4 requires k % 32 == 0, got {k}");
        if m == 0 || n == 0 {
            return;
        }
        // SAFETY: as above; offsets are checked against the buffer lengths by DevBuf::at.
        let rc = unsafe {
            lq4_gemm(
                self.ctx,
                qw.raw,
                qw_extra_offset,
                n,
                k,
                x.at(x_offset),
                LQ4_F32,
                m,
                y.at(y_offset) as *mut f32,
                ptr::null(),
                0.0,
                self.stream,
            )
        };
        check(rc).expect("lq4_gemm");
    }

    /// The projection's matmul with the adapter's delta fused into its epilogue: what a HIP caller
    /// uses instead of `dispatch_matmul` followed by `dispatch_lora_if_active`.  Falls back to the
    /// plain matmul when no adapter covers `(layer_idx, module)`.
    #[allow(clippy::too_many_arguments)]
    pub fn dispatch_matmul_with_lora(
        &self,
        x: &DevBuf,
        qw: &HipQ4WeightBuf,
        y: &DevBuf,
        m: u32,
        n: u32,
        k: u32,
        layer_idx: usize,
        module: &str,
    ) {
        assert!(k > 0 && k % 32 == 0, "dispatch_matmul_q4 requires k % 32 == 0, got {k}");
        if n == 0 || m == 0 {
            return;
        }
        let (lora, scale) = match self.projection(layer_idx, module) {
            Some((p, s)) => (p.raw as *const Lq4Lora, s),
            None => (ptr::null(), 0.0),
        };
        // SAFETY: as above.
        let rc = unsafe {
            if m <= LQ4_MAX_GEMV_BATCH {
                lq4_gemv(self.ctx, qw.raw, 0, n, k, x.ptr as *const f32, m, y.ptr as *mut f32, lora, scale, self.stream)
            } else {
                lq4_gemm(self.ctx, qw.raw, 0, n, k, x.ptr, LQ4_F32, m, y.ptr as *mut f32, lora, scale, self.stream)
            }
        };
        check(rc).expect("lq4_gemv/lq4_gemm with LoRA");
    }

    /// `dispatch_lora_if_active` (inner/layers/mod.rs:15-51): `y += scale * B (A x)` after the
    /// projection wrote y; a no-op without an adapter or without this projection, as today.
    pub fn dispatch_lora_if_active(
        &self,
        x: &DevBuf,
        x_byte_offset: u64,
        y: &DevBuf,
        y_byte_offset: u64,
        layer_idx: usize,
        module: &str,
    ) {
        let Some((proj, scale)) = self.projection(layer_idx, module) else { return };
        // SAFETY: as above.
        let rc = unsafe {
            lq4_lora_apply(self.ctx, proj.raw, scale, x.at(x_byte_offset), LQ4_F32, 1, y.at(y_byte_offset) as *mut f32, self.stream)
        };
        check(rc).expect("lq4_lora_apply");
    }

    /// `load_lora_adapter` (metal_qwen35.rs:3806-3986): same signature, same checks in the same order, same
    /// error strings; the QuaRot pre-rotation of `A` stays on the host (`rotate_adapter_for_quarot`) before upload.
    pub fn load_lora_adapter(
        &mut self,
        mut layers: Vec<LoraLayerData>,
        scale: f32,
        quarot_seed: Option<u64>,
    ) -> Result<(), String> {
        if self.lora.is_some() {
            return Err("LoRA adapter already loaded; call unload_lora_adapter first".into());
        }
        if layers.is_empty() {
            return Err("load_lora_adapter: layers must not be empty".into());
        }
        if !scale.is_finite() {
            return Err(format!("load_lora_adapter: scale must be finite, got {scale}"));
        }
        let hidden_dim = self.config.hidden_size;
        if let Some(seed) = quarot_seed {
            rotate_layers_for_quarot(&mut layers, seed, hidden_dim)?;
        }
        let num_layers = self.config.num_hidden_layers;
        let mut projections: Vec<HashMap<String, HipLoraProjection>> = (0..num_layers).map(|_| HashMap::new()).collect();
        for l in &layers {
            if l.rank == 0 {
                return Err(format!("load_lora_adapter: layer {} module '{}' has rank=0", l.layer_idx, l.module));
            }
            if l.d_in == 0 || l.d_out == 0 {
                return Err(format!(
                    "load_lora_adapter: layer {} module '{}' has zero dimension (d_in={}, d_out={})",
                    l.layer_idx, l.module, l.d_in, l.d_out
                ));
            }
            if l.layer_idx >= num_layers {
                return Err(format!("load_lora_adapter: layer_idx {} >= num_hidden_layers {}", l.layer_idx, num_layers));
            }
            let (exp_d_in, exp_d_out) = self.expected_lora_shape(l.layer_idx, &l.module)?;
            if l.d_in != exp_d_in || l.d_out != exp_d_out {
                return Err(format!(
                    "load_lora_adapter: layer {} module '{}' has (d_in={}, d_out={}) but model expects (d_in={}, d_out={})",
                    l.layer_idx, l.module, l.d_in, l.d_out, exp_d_in, exp_d_out
                ));
            }
            let expected_a = l.rank.checked_mul(l.d_in).ok_or_else(|| {
                format!("load_lora_adapter: layer {} module '{}' rank*d_in overflow", l.layer_idx, l.module)
            })?;
            let expected_b = l.d_out.checked_mul(l.rank).ok_or_else(|| {
                format!("load_lora_adapter: layer {} module '{}' d_out*rank overflow", l.layer_idx, l.module)
            })?;
            if l.a.len() != expected_a {
                return Err(format!(
                    "load_lora_adapter: layer {} module '{}' A length {} != rank*d_in {}",
                    l.layer_idx, l.module, l.a.len(), expected_a
                ));
            }
            if l.b.len() != expected_b {
                return Err(format!(
                    "load_lora_adapter: layer {} module '{}' B length {} != d_out*rank {}",
                    l.layer_idx, l.module, l.b.len(), expected_b
                ));
            }
            let rank = u32::try_from(l.rank).map_err(|_| format!("load_lora_adapter: rank {} exceeds u32", l.rank))?;
            let d_in = u32::try_from(l.d_in).map_err(|_| format!("load_lora_adapter: d_in {} exceeds u32", l.d_in))?;
            let d_out = u32::try_from(l.d_out).map_err(|_| format!("load_lora_adapter: d_out {} exceeds u32", l.d_out))?;
            if projections[l.layer_idx].contains_key(&l.module) {
                return Err(format!(
                    "load_lora_adapter: duplicate projection for layer {} module '{}'",
                    l.layer_idx, l.module
                ));
            }
            let mut raw = ptr::null_mut();
            // SAFETY: host slices live for the call; the library copies them to the device.
            check(unsafe {
                lq4_lora_upload(
                    self.ctx,
                    l.a.as_ptr() as *const c_void,
                    l.b.as_ptr() as *const c_void,
                    LQ4_F32,
                    rank,
                    d_in,
                    d_out,
                    &mut raw,
                )
            })?;
            projections[l.layer_idx].insert(l.module.clone(), HipLoraProjection { raw });
        }
        self.lora = Some(HipLoraAdapter { projections, scale });
        Ok(())
    }

    pub fn unload_lora_adapter(&mut self) {
        self.lora = None;
    }

    fn projection(&self, layer_idx: usize, module: &str) -> Option<(&HipLoraProjection, f32)> {
        let adapter = self.lora.as_ref()?;
        Some((adapter.projections.get(layer_idx)?.get(module)?, adapter.scale))
    }

    /// The GEMVs of one token between two points where the host looks at a result, as one call
    /// (`forward_step` encodes them into one command buffer, metal_qwen35.rs:6943, committed at :6447).
    pub fn encode_token_chain(&self, steps: &[Lq4ChainStep]) {
        assert!(steps.len() <= LQ4_CHAIN_MAX_STEPS, "a chain holds at most {LQ4_CHAIN_MAX_STEPS} steps");
        if steps.is_empty() {
            return;
        }
        // SAFETY: steps points at steps.len() initialised descriptors.
        check(unsafe { lq4_gemv_chain(self.ctx, steps.as_ptr(), steps.len() as u32, self.stream) }).expect("lq4_gemv_chain");
    }

    /// The MoE FFN of one layer for `tokens` rows of `x` (`encode_moe_ffn`, inner/layers/mod.rs:226-660;
    /// CPU form `moe_ffn_step`, model/qwen35/moe.rs:8-36): router softmax / top-k / renormalise from the
    /// router logits, the routed experts, and the always-active shared expert onto the same `y`, as one
    /// library call.  Unlike the Metal path nothing is read back to the host between the steps (the
    /// router and the shared expert's sigmoid gate stay on the device).
    pub fn encode_moe_ffn(&self, router_logits: &DevBuf, moe: &HipMoeLayer, x: &DevBuf, tokens: u32, y: &DevBuf) {
        // SAFETY: the buffers hold [tokens, E] logits and [tokens, hidden] activations and outputs; the
        // weight handles were uploaded with these shapes.
        check(unsafe {
            lq4_moe_ffn(
                self.ctx, router_logits.ptr as *const f32, moe.gate_up.raw, moe.down.raw, moe.num_experts, moe.top_k,
                moe.inter, moe.shared_gate_up.raw, moe.shared_down.raw, moe.shared_expert_gate.ptr as *const f32,
                moe.shared_inter, moe.hidden, x.ptr as *const f32, tokens, y.ptr as *mut f32, self.stream,
            )
        })
        .expect("lq4_moe_ffn");
    }

    /// `commit()` + `wait_until_completed()` of the command buffer.
    pub fn synchronize(&self) -> Result<(), String> {
        // SAFETY: plain call.
        check(unsafe { lq4_sync(self.ctx, self.stream) })
    }
}

/// The host-side QuaRot rotation of the factors before upload, exactly the call the Metal backend
/// makes (metal_qwen35.rs:3834-3849); `hidden_dim` comes from the model config.
fn rotate_layers_for_quarot(layers: &mut [LoraLayerData], seed: u64, hidden_dim: usize) -> Result<(), String> {
    use crate::quant::quarot::lora::{rotate_adapter_for_quarot, LoraLayerMut};
    use crate::quant::quarot::plan::RotationPlan;
    let plan = RotationPlan::qwen35_residual_stream_linear_layers();
    let lora_muts: Vec<LoraLayerMut<'_>> = layers
        .iter_mut()
        .map(|l| LoraLayerMut {
            layer_idx: l.layer_idx,
            module: &l.module,
            a: &mut l.a,
            b: &mut l.b,
            rank: l.rank,
            d_in: l.d_in,
            d_out: l.d_out,
        })
        .collect();
    rotate_adapter_for_quarot(lora_muts, seed, hidden_dim, &plan).map_err(|e| e.to_string())
}
