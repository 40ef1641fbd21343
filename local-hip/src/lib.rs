//! HIP (MI355X / gfx950) backend behind the kernel-dispatch API that `local-engine` calls on `local-metal`.
//!
//! `ffi` holds the raw declarations of `liblocal_hip.so` (generated from `include/local_hip.h`).  The safe layer
//! with the reference's type and method names (`Context`, `Buffer`, `CommandBatch`, `Kernels::<op>_into`, and an
//! `Error` enum with the variants of `local_metal::Error`) wraps them one to one.
pub mod ffi;

use core::ffi::CStr;

/// Message of the last failed call on this thread (`lh_last_error`), in the wording of `local_metal::Error`'s
/// `Display` (local-metal/src/error.rs:1-32).
pub fn last_error() -> String {
    // SAFETY: lh_last_error returns a pointer to a NUL-terminated thread-local buffer that stays valid until the
    // next failing call on this thread.
    unsafe { CStr::from_ptr(ffi::lh_last_error()) }.to_string_lossy().into_owned()
}
