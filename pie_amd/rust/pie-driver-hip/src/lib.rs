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
/// The C side accepts NULL (no notification), hence `Option<ReadyCb>` in the signatures.
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
        ready_cb: Option<ReadyCb>,
        ready_ctx: *mut c_void,
        vtable: InProcVTable,
    ) -> c_int;
    /// Stops every live instance of this flavour; callable from any thread, also while an
    /// instance is still loading its model.
    pub fn pie_driver_hip_request_stop();
}

/// Raw declarations and constants of the kernel library, generated from
/// `include/pie_hip_kernels.h` by `gen_sys.py` (every entry point, every `PIE_HIP_*` constant).
pub mod sys;
pub use sys::*;

/// Refuses a kernel library whose ABI version differs from the header these bindings were
/// generated from: an older or newer library links, and then computes garbage.
pub fn check_abi() -> Result<(), KernelError> {
    if unsafe { pie_hip_abi_version() } == PIE_HIP_ABI_VERSION { Ok(()) } else { Err(KernelError::AbiMismatch) }
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
    /// The loaded library's `pie_hip_abi_version()` is not `PIE_HIP_ABI_VERSION`.
    AbiMismatch,
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
    ready_cb: Option<ReadyCb>,
    ready_ctx: *mut c_void,
    vtable: InProcVTable,
) -> Result<(), c_int> {
    check_abi().map_err(|_| -2)?;
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
