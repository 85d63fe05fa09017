//! FFI surface of the MI355X (HIP) Pie driver.
//!
//! Two layers, both plain C ABIs with no C++ types in their signatures:
//!
//! * the runtime-facing pair every driver flavour exports — `pie_driver_hip_run_inproc` and
//!   `pie_driver_hip_request_stop` (`include/pie_driver_abi.h`) — which the server binds next to
//!   its `portable` and `cuda` flavours (`server/src/driver_ffi.rs:18-46,205-257` in the Pie tree);
//! * the kernel library below the driver (`include/pie_hip_kernels.h`): one function per fused
//!   operator, device pointers + shapes + a `hipStream_t`, an `int` status, no allocation.
//!
//! NOTE: this file was written without a Rust toolchain available and has never been compiled.
//! The declarations follow the C headers field for field; `tests/test_abi_layout.py` checks the
//! C side of the descriptor layouts against the reference bridge header.

#![allow(non_camel_case_types)]

use std::ffi::{c_char, c_int, c_void, CStr};

/// `void (*ready_cb)(const char* caps_json, void* ctx)`: called once, after weights and the KV
/// pool are allocated, with the capabilities JSON.
pub type ReadyCb = unsafe extern "C" fn(caps_json: *const c_char, ctx: *mut c_void);

/// `PieInProcVTable` (`driver/bridge/include/pie_bridge.h:437-451`), passed by value.
#[repr(C)]
#[derive(Copy, Clone)]
pub struct InProcVTable {
    /// 0 = a frame (or none yet when `*out` stays null), -1 = clean shutdown, other = error.
    pub recv: unsafe extern "C" fn(ctx: *mut c_void, out: *mut *const c_void, req_id: *mut u32) -> i32,
    /// The callee copies synchronously; the response slices belong to the driver.
    pub send_response: unsafe extern "C" fn(ctx: *mut c_void, req_id: u32, resp: *const c_void),
    pub ctx: *mut c_void,
}

extern "C" {
    /// Blocks until the serve loop exits.  0, or -1 on any failure; no exception crosses.
    pub fn pie_driver_hip_run_inproc(
        argc: c_int,
        argv: *mut *mut c_char,
        install_signal_handlers: c_int,
        ready_cb: ReadyCb,
        ready_ctx: *mut c_void,
        vtable: InProcVTable,
    ) -> c_int;
    /// Stops every live instance of this flavour; callable from any thread, also while an
    /// instance is still loading its model.
    pub fn pie_driver_hip_request_stop();
}

/// Status codes of the kernel library.
pub const PIE_HIP_OK: c_int = 0;
pub const PIE_HIP_ERR_INVALID: c_int = 1;
pub const PIE_HIP_ERR_UNSUPPORTED: c_int = 2;
pub const PIE_HIP_ERR_LAUNCH: c_int = 3;

/// Weight storage formats (`format` arguments).
pub const PIE_HIP_FMT_INT4B8: c_int = 0;
pub const PIE_HIP_FMT_INT8: c_int = 1;
pub const PIE_HIP_FMT_FP8: c_int = 2;
pub const PIE_HIP_FMT_BF16: c_int = 3;

/// KV-cache storage formats (`kv_format` arguments).
pub const PIE_HIP_KV_BF16: c_int = 0;
pub const PIE_HIP_KV_FP8_E4M3: c_int = 1;
pub const PIE_HIP_KV_INT8_PER_TOKEN_HEAD: c_int = 2;
pub const PIE_HIP_KV_FP8_PER_TOKEN_HEAD: c_int = 3;
pub const PIE_HIP_KV_FP8_E5M2: c_int = 4;

/// RoPE pairings of the rotation kernels and fused epilogues.
pub const PIE_HIP_ROPE_HALF: c_int = 0;
pub const PIE_HIP_ROPE_ADJACENT: c_int = 1;
pub const PIE_HIP_ROPE_HALF_PAIRED_ROWS: c_int = 2;

extern "C" {
    pub fn pie_hip_abi_version() -> c_int;

    // ---- quantised linears -------------------------------------------------------------------
    pub fn pie_hip_linear_fused(
        format: c_int, act_bf16: *const u16, norm_weight_bf16: *const u16, eps: f32,
        weight: *const c_void, scale: *const c_void, scale_is_bf16: c_int, group_size: c_int,
        y_bf16: *mut u16, m: c_int, n: c_int, k: c_int, beta: c_int, swiglu: c_int,
        stream: *mut c_void,
    ) -> c_int;
    pub fn pie_hip_qkv_rope_fused(
        format: c_int, act_bf16: *const u16, norm_weight_bf16: *const u16, eps: f32,
        weight: *const c_void, scale: *const c_void, scale_is_bf16: c_int, group_size: c_int,
        m: c_int, k: c_int, rope_table: *const f32, kv_slots: *const i64, q_out: *mut u16,
        k_pages: *mut u16, v_pages: *mut u16, num_q_heads: c_int, num_kv_heads: c_int,
        head_dim: c_int, pairing: c_int, stream: *mut c_void,
    ) -> c_int;
    pub fn pie_hip_gemm_skinny_tiled(
        format: c_int, act_bf16: *const u16, weight: *const c_void, scale: *const c_void,
        scale_is_bf16: c_int, group_size: c_int, y_bf16: *mut u16, m: c_int, n: c_int, k: c_int,
        beta: c_int, swiglu: c_int, stream: *mut c_void,
    ) -> c_int;
    pub fn pie_hip_gemm_mfma(
        format: c_int, act_bf16: *const u16, weight: *const c_void, scale: *const c_void,
        scale_is_bf16: c_int, group_size: c_int, y_bf16: *mut u16, m: c_int, n: c_int, k: c_int,
        beta: c_int, swiglu: c_int, stream: *mut c_void,
    ) -> c_int;
    pub fn pie_hip_lm_head_argmax_workspace_bytes(m: c_int, v: c_int) -> usize;
    pub fn pie_hip_lm_head_argmax(
        act_bf16: *const u16, norm_weight_bf16: *const u16, eps: f32, w_bf16: *const u16,
        logits_bf16: *mut u16, out_tokens: *mut u32, m: c_int, v: c_int, h: c_int,
        workspace: *mut c_void, workspace_bytes: usize, stream: *mut c_void,
    ) -> c_int;

    // ---- paged attention ----------------------------------------------------------------------
    pub fn pie_hip_attn_decode_workspace_bytes(
        num_requests: c_int, num_q_heads: c_int, num_kv_heads: c_int, head_dim: c_int,
        max_kv_len: c_int,
    ) -> usize;
    pub fn pie_hip_attn_rows_paged(
        q: *const u16, k_pages: *const u16, v_pages: *const u16, o: *mut u16, lse: *mut f32,
        kv_page_indices: *const u32, row_page_begin: *const u32, row_kv_len: *const i32,
        num_rows: c_int, num_q_heads: c_int, num_kv_heads: c_int, head_dim: c_int,
        page_size: c_int, sm_scale: f32, max_kv_len: c_int, workspace: *mut c_void,
        workspace_bytes: usize, stream: *mut c_void,
    ) -> c_int;
    /// The same without a workspace or any allocation (split partials in a 16 MiB device array
    /// built into the library); larger batches return `PIE_HIP_ERR_UNSUPPORTED`.
    pub fn pie_hip_attn_rows_paged_static(
        q: *const u16, k_pages: *const u16, v_pages: *const u16, o: *mut u16, lse: *mut f32,
        kv_page_indices: *const u32, row_page_begin: *const u32, row_kv_len: *const i32,
        num_rows: c_int, num_q_heads: c_int, num_kv_heads: c_int, head_dim: c_int,
        page_size: c_int, sm_scale: f32, max_kv_len: c_int, stream: *mut c_void,
    ) -> c_int;
    pub fn pie_hip_attn_rows_paged_kvq(
        kv_format: c_int, q: *const u16, k_pages: *const c_void, v_pages: *const c_void,
        k_scales: *const f32, v_scales: *const f32, o: *mut u16, lse: *mut f32,
        kv_page_indices: *const u32, row_page_begin: *const u32, row_kv_len: *const i32,
        num_rows: c_int, num_q_heads: c_int, num_kv_heads: c_int, head_dim: c_int,
        page_size: c_int, sm_scale: f32, max_kv_len: c_int, workspace: *mut c_void,
        workspace_bytes: usize, stream: *mut c_void,
    ) -> c_int;
    pub fn pie_hip_kv_write_quant(
        kv_format: c_int, k_rows: *const u16, v_rows: *const u16, kv_slots: *const i64,
        k_pages: *mut c_void, v_pages: *mut c_void, k_scales: *mut f32, v_scales: *mut f32,
        num_tokens: c_int, num_kv_heads: c_int, head_dim: c_int, page_size: c_int,
        stream: *mut c_void,
    ) -> c_int;
    pub fn pie_hip_kv_dequant_pages(
        kv_format: c_int, k_pages: *const c_void, v_pages: *const c_void, k_scales: *const f32,
        v_scales: *const f32, k_out: *mut u16, v_out: *mut u16, page_ids: *const u32,
        num_pages: c_int, num_kv_heads: c_int, head_dim: c_int, page_size: c_int,
        stream: *mut c_void,
    ) -> c_int;

    // ---- layer ops ------------------------------------------------------------------------------
    pub fn pie_hip_embed(
        token_ids: *const u32, table_bf16: *const u16, y_bf16: *mut u16, num_tokens: c_int,
        hidden: c_int, vocab: c_int, stream: *mut c_void,
    ) -> c_int;
    pub fn pie_hip_rmsnorm(
        x_bf16: *const u16, weight_bf16: *const u16, y_bf16: *mut u16, num_tokens: c_int,
        hidden: c_int, eps: f32, stream: *mut c_void,
    ) -> c_int;
    pub fn pie_hip_rope_table(
        positions: *const i32, inv_freq: *const f32, table: *mut f32, num_tokens: c_int,
        head_dim: c_int, stream: *mut c_void,
    ) -> c_int;
    pub fn pie_hip_argmax(
        logits_bf16: *const u16, out_idx: *mut u32, rows: c_int, vocab: c_int, stream: *mut c_void,
    ) -> c_int;
    pub fn pie_hip_copy_kv_pages(
        pool: *mut c_void, src_pages: *const u32, dst_pages: *const u32, num_pairs: c_int,
        page_bytes: usize, stream: *mut c_void,
    ) -> c_int;
}

/// A kernel-library status as a `Result`.
pub fn check(status: c_int) -> Result<(), KernelError> {
    match status {
        PIE_HIP_OK => Ok(()),
        PIE_HIP_ERR_INVALID => Err(KernelError::InvalidArgument),
        PIE_HIP_ERR_UNSUPPORTED => Err(KernelError::UnsupportedShape),
        _ => Err(KernelError::Launch),
    }
}

#[derive(Copy, Clone, Debug, Eq, PartialEq)]
pub enum KernelError {
    InvalidArgument,
    UnsupportedShape,
    Launch,
}

/// Runs the driver on the calling thread, the way the server's flavour dispatcher does for the
/// other in-process drivers: `args` are the program name followed by `--config <file.toml>`.
///
/// # Safety
/// `vtable`'s callbacks and context must stay valid until this returns; `ready_ctx` is handed
/// back to `ready_cb` unchanged.
pub unsafe fn run_inproc(
    args: &[&CStr],
    install_signal_handlers: bool,
    ready_cb: ReadyCb,
    ready_ctx: *mut c_void,
    vtable: InProcVTable,
) -> Result<(), c_int> {
    let mut argv: Vec<*mut c_char> = args.iter().map(|a| a.as_ptr() as *mut c_char).collect();
    let rc = pie_driver_hip_run_inproc(
        argv.len() as c_int,
        argv.as_mut_ptr(),
        install_signal_handlers as c_int,
        ready_cb,
        ready_ctx,
        vtable,
    );
    if rc == 0 { Ok(()) } else { Err(rc) }
}

/// Asks every live HIP driver instance of this process to leave its serve loop.
pub fn request_stop() {
    unsafe { pie_driver_hip_request_stop() }
}
