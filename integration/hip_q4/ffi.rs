//! Raw bindings of `liblattice_hip_q4.so` (`include/lattice_hip_q4.h`), one declaration per exported
//! symbol.  Meant to live at `crates/inference/src/forward/hip_q4/ffi.rs` behind a `hip-gpu` feature
//! (`#[cfg(feature = "hip-gpu")] mod hip_q4;` next to the `metal-gpu` arm).  `build.rs` adds
//! `cargo:rustc-link-lib=dylib=lattice_hip_q4` and a `rustc-link-search` to the directory holding the
//! library; at run time ROCm's `libamdhip64.so` must be on the loader path.
//!
//! Not compiled here (the build image has no `rustc`); every signature is checked against the header
//! by eye and against `lattice_amd/backend.py`, the ctypes binding of the same symbols that the test
//! suite drives.
#![allow(non_camel_case_types, dead_code)]

use std::os::raw::{c_char, c_int, c_void};

/// Opaque handles (`lq4_ctx`, `lq4_weight`, `lq4_lora`).
#[repr(C)]
pub struct Lq4Ctx {
    _p: [u8; 0],
}
#[repr(C)]
pub struct Lq4Weight {
    _p: [u8; 0],
}
#[repr(C)]
pub struct Lq4Lora {
    _p: [u8; 0],
}

// status codes
pub const LQ4_OK: c_int = 0;
pub const LQ4_E_INVALID: c_int = -1;
pub const LQ4_E_HIP: c_int = -2;
pub const LQ4_E_BLOCK: c_int = -3;
pub const LQ4_E_NOMEM: c_int = -4;
pub const LQ4_E_UNSUPPORTED: c_int = -5;
pub const LQ4_MAX_LORA_RANK: u32 = 64;
pub const LQ4_MAX_GEMV_BATCH: u32 = 16;

// activation / factor dtypes
pub const LQ4_F32: c_int = 0;
pub const LQ4_F16: c_int = 1;

// lq4_gemv_fusion / lq4_chain_step
pub const LQ4_PRO_NONE: c_int = 0;
pub const LQ4_PRO_ADD_RMSNORM: c_int = 1;
pub const LQ4_PRO_SILU_MUL: c_int = 2;
pub const LQ4_EPI_NONE: c_int = 0;
pub const LQ4_EPI_ADD_RESIDUAL: c_int = 1;
pub const LQ4_EPI_SILU_MUL_PAIRS: c_int = 2;
pub const LQ4_CHAIN_MAX_STEPS: usize = 16;
pub const LQ4_MAX_TOP_K: u32 = 256;
pub const LQ4_STATIC_SCRATCH_BYTES: usize = 2 << 20;

/// `lq4_gemv_fusion`: the elementwise steps around a one-token GEMV
/// (`dispatch_fused_residual_add_norm`, `dispatch_silu_mul_fused`, `dispatch_add_and_copy`).
#[repr(C)]
#[derive(Clone, Copy)]
pub struct Lq4GemvFusion {
    pub prologue: c_int,
    pub base: *const f32,
    pub delta: *const f32, // may be null
    pub gamma: *const f32,
    pub eps: f32,
    pub residual_out: *mut f32, // may be null; must not overlap base or delta
    pub epilogue: c_int,
    pub residual: *mut f32,
    pub copy_dst: *mut f32, // may be null
}

/// `lq4_chain_step`: one GEMV of a token's chain (`forward_step` encodes them into one command buffer).
#[repr(C)]
#[derive(Clone, Copy)]
pub struct Lq4ChainStep {
    pub w: *const Lq4Weight,
    pub w_extra_offset: u64,
    pub n: u32,
    pub k: u32,
    pub from_previous: c_int,
    pub x_dev: *const f32,
    pub prologue: c_int,
    pub base: *const f32,
    pub delta: *const f32,
    pub gamma: *const f32,
    pub eps: f32,
    pub residual_out: *mut f32,
    pub epilogue: c_int,
    pub residual: *mut f32,
    pub y_dev: *mut f32,
}

/// `lq4_path_counters`: which kernels served the calls of a context (tests, diagnostics).
#[repr(C)]
#[derive(Clone, Copy, Default, Debug)]
pub struct Lq4PathCounters {
    pub gemv: u64,
    pub gemm: u64,
    pub lora_a: u64,
    pub moe_route: u64,
    pub moe_gate_up: u64,
    pub moe_down: u64,
    pub dequant: u64,
    pub topk: u64,
    pub gemv_fused: u64,
    pub elementwise: u64,
    pub gemv_chain: u64,
    pub lora_t_fallback: u64,
    pub gemv_multi: u64,
}

/// One weight view of `lq4_gemv_multi` with its output and optional adapter.
#[repr(C)]
pub struct Lq4Projection {
    pub w: *const Lq4Weight,
    pub w_extra_offset: u64,
    pub n: u32,
    pub y_dev: *mut f32,
    pub lora: *const Lq4Lora,
    pub lora_scale: f32,
}
pub const LQ4_MAX_PROJECTIONS: usize = 8;

#[link(name = "lattice_hip_q4")]
extern "C" {
    pub fn lq4_last_error() -> *const c_char;
    pub fn lq4_version() -> *const c_char;
    pub fn lq4_ctx_create(device_ordinal: c_int, out: *mut *mut Lq4Ctx) -> c_int;
    pub fn lq4_ctx_destroy(ctx: *mut Lq4Ctx) -> c_int;
    pub fn lq4_ctx_reserve_scratch(ctx: *mut Lq4Ctx, bytes: usize) -> c_int;
    pub fn lq4_sync(ctx: *mut Lq4Ctx, stream: *mut c_void) -> c_int;

    // ---- Q4 weights: upload, residency, ingress rule
    pub fn lq4_validate_blocks(payload: *const u8, nbytes: usize, bad_block: *mut i64, reason: *mut c_int) -> c_int;
    pub fn lq4_weight_upload(
        ctx: *mut Lq4Ctx,
        bytes: *const u8,
        nbytes: usize,
        payload_offset: u64,
        validate: c_int,
        out: *mut *mut Lq4Weight,
    ) -> c_int;
    pub fn lq4_weight_wrap(
        ctx: *mut Lq4Ctx,
        dev: *const c_void,
        nbytes: usize,
        payload_offset: u64,
        out: *mut *mut Lq4Weight,
    ) -> c_int;
    pub fn lq4_weight_free(w: *mut Lq4Weight) -> c_int;
    pub fn lq4_weight_info(
        w: *const Lq4Weight,
        base_dev: *mut *const c_void,
        nbytes: *mut usize,
        payload_offset: *mut u64,
    ) -> c_int;

    // ---- LoRA
    pub fn lq4_lora_upload(
        ctx: *mut Lq4Ctx,
        a: *const c_void,
        b: *const c_void,
        dtype: c_int,
        rank: u32,
        d_in: u32,
        d_out: u32,
        out: *mut *mut Lq4Lora,
    ) -> c_int;
    pub fn lq4_lora_free(l: *mut Lq4Lora) -> c_int;
    pub fn lq4_lora_apply(
        ctx: *mut Lq4Ctx,
        l: *const Lq4Lora,
        lora_scale: f32,
        x: *const c_void,
        x_dtype: c_int,
        rows: u32,
        y: *mut f32,
        stream: *mut c_void,
    ) -> c_int;

    // ---- decode GEMV, prefill GEMM (optional fused LoRA: pass null for none)
    pub fn lq4_gemv(
        ctx: *mut Lq4Ctx,
        w: *const Lq4Weight,
        w_extra_offset: u64,
        n: u32,
        k: u32,
        x: *const f32,
        batch: u32,
        y: *mut f32,
        lora: *const Lq4Lora,
        lora_scale: f32,
        stream: *mut c_void,
    ) -> c_int;
    /// Several projections of one x: one launch at batch 1 (q, k, v of gqa.rs:72-127 without a merged file).
    pub fn lq4_gemv_multi(
        ctx: *mut Lq4Ctx,
        proj: *const Lq4Projection,
        count: u32,
        k: u32,
        x: *const f32,
        batch: u32,
        stream: *mut c_void,
    ) -> c_int;
    pub fn lq4_gemm(
        ctx: *mut Lq4Ctx,
        w: *const Lq4Weight,
        w_extra_offset: u64,
        n: u32,
        k: u32,
        x: *const c_void,
        x_dtype: c_int,
        m: u32,
        y: *mut f32,
        lora: *const Lq4Lora,
        lora_scale: f32,
        stream: *mut c_void,
    ) -> c_int;
    pub fn lq4_gemv_fused(
        ctx: *mut Lq4Ctx,
        w: *const Lq4Weight,
        w_extra_offset: u64,
        n: u32,
        k: u32,
        x: *const f32,
        y: *mut f32,
        fusion: *const Lq4GemvFusion,
        lora: *const Lq4Lora,
        lora_scale: f32,
        stream: *mut c_void,
    ) -> c_int;
    pub fn lq4_gemv_fused_batch(
        ctx: *mut Lq4Ctx,
        w: *const Lq4Weight,
        w_extra_offset: u64,
        n: u32,
        k: u32,
        x: *const f32,
        batch: u32,
        y: *mut f32,
        fusion: *const Lq4GemvFusion,
        lora: *const Lq4Lora,
        lora_scale: f32,
        stream: *mut c_void,
    ) -> c_int;

    // ---- MoE
    pub fn lq4_moe_route(
        ctx: *mut Lq4Ctx,
        logits: *const f32,
        tokens: u32,
        num_experts: u32,
        top_k: u32,
        ids: *mut i32,
        weights: *mut f32,
        stream: *mut c_void,
    ) -> c_int;
    pub fn lq4_moe_grouped_gemv(
        ctx: *mut Lq4Ctx,
        gate_up: *const Lq4Weight,
        down: *const Lq4Weight,
        num_experts: u32,
        inter: u32,
        hidden: u32,
        x: *const f32,
        tokens: u32,
        ids: *const i32,
        weights: *const f32,
        top_k: u32,
        y: *mut f32,
        stream: *mut c_void,
    ) -> c_int;
    pub fn lq4_moe_shared_expert(
        ctx: *mut Lq4Ctx,
        gate_up: *const Lq4Weight,
        down: *const Lq4Weight,
        shared_gate: *const f32,
        shared_inter: u32,
        hidden: u32,
        x: *const f32,
        tokens: u32,
        y: *mut f32,
        stream: *mut c_void,
    ) -> c_int;

    pub fn lq4_moe_ffn(
        ctx: *mut Lq4Ctx,
        router_logits: *const f32,
        gate_up: *const Lq4Weight,
        down: *const Lq4Weight,
        num_experts: u32,
        top_k: u32,
        inter: u32,
        shared_gate_up: *const Lq4Weight,
        shared_down: *const Lq4Weight,
        shared_gate: *const f32,
        shared_inter: u32,
        hidden: u32,
        x: *const f32,
        tokens: u32,
        y: *mut f32,
        stream: *mut c_void,
    ) -> c_int;

    // ---- lm_head and top-k
    pub fn lq4_topk(
        ctx: *mut Lq4Ctx,
        logits: *const f32,
        n: u32,
        top_k: u32,
        out_logits: *mut f32,
        out_ids: *mut u32,
        stream: *mut c_void,
    ) -> c_int;
    pub fn lq4_lm_head_topk(
        ctx: *mut Lq4Ctx,
        w: *const Lq4Weight,
        w_extra_offset: u64,
        vocab: u32,
        k: u32,
        x: *const f32,
        top_k: u32,
        out_logits: *mut f32,
        out_ids: *mut u32,
        stream: *mut c_void,
    ) -> c_int;
    /// The same for callers that may not allocate device memory (scratch in a static device array).
    pub fn lq4_lm_head_topk_static(
        ctx: *mut Lq4Ctx,
        w: *const Lq4Weight,
        w_extra_offset: u64,
        vocab: u32,
        k: u32,
        x: *const f32,
        top_k: u32,
        out_logits: *mut f32,
        out_ids: *mut u32,
        stream: *mut c_void,
    ) -> c_int;

    // ---- elementwise steps
    pub fn lq4_residual_add_rmsnorm(
        ctx: *mut Lq4Ctx,
        base: *const f32,
        delta: *const f32,
        gamma: *const f32,
        hidden: u32,
        rows: u32,
        eps: f32,
        residual_out: *mut f32,
        normed_out: *mut f32,
        stream: *mut c_void,
    ) -> c_int;
    pub fn lq4_silu_mul(
        ctx: *mut Lq4Ctx,
        gate_up: *const f32,
        count: u32,
        rows: u32,
        out: *mut f32,
        out_stride: u32,
        stream: *mut c_void,
    ) -> c_int;
    pub fn lq4_add_and_copy(
        ctx: *mut Lq4Ctx,
        src: *const f32,
        residual: *mut f32,
        dst: *mut f32,
        count: usize,
        stream: *mut c_void,
    ) -> c_int;

    // ---- sibling block formats
    pub fn lq4_gemv_q8(
        ctx: *mut Lq4Ctx,
        w: *const Lq4Weight,
        w_extra_offset: u64,
        n: u32,
        k: u32,
        x: *const f32,
        batch: u32,
        y: *mut f32,
        stream: *mut c_void,
    ) -> c_int;
    pub fn lq4_gemm_q8(
        ctx: *mut Lq4Ctx,
        w: *const Lq4Weight,
        w_extra_offset: u64,
        n: u32,
        k: u32,
        x: *const c_void,
        x_dtype: c_int,
        m: u32,
        y: *mut f32,
        stream: *mut c_void,
    ) -> c_int;
    pub fn lq4_gemv_q3(
        ctx: *mut Lq4Ctx,
        w: *const Lq4Weight,
        w_extra_offset: u64,
        n: u32,
        k: u32,
        x: *const f32,
        batch: u32,
        y: *mut f32,
        stream: *mut c_void,
    ) -> c_int;
    pub fn lq4_gemm_q3(
        ctx: *mut Lq4Ctx,
        w: *const Lq4Weight,
        w_extra_offset: u64,
        n: u32,
        k: u32,
        x: *const c_void,
        x_dtype: c_int,
        m: u32,
        y: *mut f32,
        stream: *mut c_void,
    ) -> c_int;

    // ---- probes, tuning hooks, counters
    pub fn lq4_dequant(
        ctx: *mut Lq4Ctx,
        w: *const Lq4Weight,
        w_extra_offset: u64,
        n: u32,
        k: u32,
        out: *mut f32,
        stream: *mut c_void,
    ) -> c_int;
    pub fn lq4_probe_read(ctx: *mut Lq4Ctx, p: *const c_void, nbytes: usize, stream: *mut c_void) -> c_int;
    pub fn lq4_probe_read_config(
        ctx: *mut Lq4Ctx,
        p: *const c_void,
        nbytes: usize,
        workgroups: u32,
        bytes_in_flight: u32,
        strided: c_int,
        nontemporal: c_int,
        stream: *mut c_void,
    ) -> c_int;
    pub fn lq4_probe_copy(ctx: *mut Lq4Ctx, src: *const c_void, dst: *mut c_void, nbytes: usize, stream: *mut c_void) -> c_int;
    /// 0 = by shape, 1 = lane-owns-block kernel, 2 = LDS-ring kernel wherever the shape fits.
    pub fn lq4_set_gemv_kernel(ctx: *mut Lq4Ctx, which: c_int) -> c_int;
    pub fn lq4_set_gemm_kernel(ctx: *mut Lq4Ctx, which: c_int) -> c_int;
    pub fn lq4_get_path_counters(ctx: *const Lq4Ctx, out: *mut Lq4PathCounters) -> c_int;

    // ---- device memory for callers without a HIP binding of their own
    pub fn lq4_malloc(ctx: *mut Lq4Ctx, nbytes: usize, out: *mut *mut c_void) -> c_int;
    pub fn lq4_free(ctx: *mut Lq4Ctx, p: *mut c_void) -> c_int;
    pub fn lq4_memcpy_h2d(ctx: *mut Lq4Ctx, dst: *mut c_void, src: *const c_void, nbytes: usize) -> c_int;
    pub fn lq4_memcpy_d2h(ctx: *mut Lq4Ctx, dst: *mut c_void, src: *const c_void, nbytes: usize) -> c_int;
}

/// `Ok(())` for `LQ4_OK`, otherwise the library's message for the calling thread
/// (the reference's loaders return `Result<_, String>`: `mmap_q4_weight`, metal_qwen35.rs:660-702).
pub fn check(rc: c_int) -> Result<(), String> {
    if rc == LQ4_OK {
        return Ok(());
    }
    // SAFETY: lq4_last_error returns a NUL-terminated string owned by the library, valid until the
    // next failing call on this thread.
    let msg = unsafe { std::ffi::CStr::from_ptr(lq4_last_error()) }
        .to_string_lossy()
        .into_owned();
    Err(format!("lattice_hip_q4 error {rc}: {msg}"))
}
