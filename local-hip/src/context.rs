//! `Context`: one gfx950 device and one in-order stream -- the role `MetalContext` (device + command queue,
//! local-metal/src/context.rs:31-104) has in the reference.
use core::ffi::c_char;
use core::ptr;

use crate::error::{check, Result};
use crate::ffi;

pub struct Context {
    raw: *mut ffi::lh_context,
}

// The library serialises nothing for the caller: a context and everything created from it belong to one thread at a
// time, as a MetalContext's queue does in the reference's single GPU worker (cli/serve.rs:603).
unsafe impl Send for Context {}

impl Context {
    /// `MetalContext::new()`: device 0.
    pub fn new() -> Result<Self> {
        Self::with_device(0)
    }

    pub fn with_device(device_index: i32) -> Result<Self> {
        let mut raw = ptr::null_mut();
        // SAFETY: `raw` is a valid out pointer; the library fills it only on success.
        check(unsafe { ffi::lh_context_create(device_index, &mut raw) })?;
        Ok(Context { raw })
    }

    /// `MetalContext::device_name()` (context.rs:58).
    pub fn device_name(&self) -> String {
        let mut buf = [0 as c_char; 256];
        // SAFETY: the buffer is writable for its length and the library NUL-terminates within it.
        if unsafe { ffi::lh_context_device_name(self.raw, buf.as_mut_ptr(), buf.len()) } != ffi::LH_OK {
            return String::new();
        }
        // SAFETY: NUL-terminated by the call above.
        unsafe { core::ffi::CStr::from_ptr(buf.as_ptr()) }.to_string_lossy().into_owned()
    }

    /// Compute units of the device (the nearest thing to `DeviceCaps`, context.rs:16-29, that matters for launch shapes).
    pub fn compute_units(&self) -> i32 {
        // SAFETY: live handle.
        unsafe { ffi::lh_context_compute_units(self.raw) }
    }

    /// Waits for everything enqueued on the context's stream; reports GPU errors and kernel-reported faults.
    pub fn synchronize(&self) -> Result<()> {
        // SAFETY: live handle.
        check(unsafe { ffi::lh_context_synchronize(self.raw) })
    }

    pub fn as_ptr(&self) -> *mut ffi::lh_context {
        self.raw
    }
}

impl Drop for Context {
    fn drop(&mut self) {
        // SAFETY: created by lh_context_create; buffers and batches hold references of their own, so the order of drops
        // does not matter.
        unsafe { ffi::lh_context_destroy(self.raw) }
    }
}
