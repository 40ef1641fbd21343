//! `Buffer`: device memory behind the method names of `MetalBuffer` (local-metal/src/buffer.rs:17-140).  A MetalBuffer
//! is CPU-visible shared memory, so the reference reads and writes it through slices; HBM is not host-visible, so
//! `as_slice` becomes `to_vec` (a copy) and writes go through `copy_from_bytes`.
use core::ffi::c_void;
use core::mem::size_of;
use core::ptr;

use crate::context::Context;
use crate::error::{check, Result};
use crate::ffi;

pub struct Buffer {
    raw: *mut ffi::lh_buffer,
}

unsafe impl Send for Buffer {}

impl Buffer {
    /// `MetalBuffer::from_slice(device, data)` (buffer.rs:28-52): a device copy of `data`.
    pub fn from_slice<T: Copy>(ctx: &Context, data: &[T]) -> Result<Self> {
        let mut raw = ptr::null_mut();
        // SAFETY: `data` is readable for its byte length; the copy completes before the call returns.
        check(unsafe { ffi::lh_buffer_from_bytes(ctx.as_ptr(), data.as_ptr() as *const c_void, data.len() * size_of::<T>(), &mut raw) })?;
        Ok(Buffer { raw })
    }

    /// `MetalBuffer::empty(device, byte_len)` (buffer.rs:54-64): zero-filled.
    pub fn empty(ctx: &Context, byte_len: usize) -> Result<Self> {
        let mut raw = ptr::null_mut();
        // SAFETY: valid out pointer.
        check(unsafe { ffi::lh_buffer_empty(ctx.as_ptr(), byte_len, &mut raw) })?;
        Ok(Buffer { raw })
    }

    /// A non-owning window of `len` bytes at `offset` (the reference passes byte offsets into one large buffer where this
    /// API takes a buffer; a view gives such a call its operand).
    pub fn view(&self, offset: usize, len: usize) -> Result<Buffer> {
        let mut raw = ptr::null_mut();
        // SAFETY: live parent handle; the library checks the range.
        check(unsafe { ffi::lh_buffer_view(self.raw, offset, len, &mut raw) })?;
        Ok(Buffer { raw })
    }

    /// `MetalBuffer::length()` (buffer.rs:66): bytes.
    pub fn length(&self) -> usize {
        // SAFETY: live handle.
        unsafe { ffi::lh_buffer_length(self.raw) }
    }

    /// What `as_slice::<T>()` (buffer.rs:78-92) gives the reference, as a host copy; waits for the stream first.
    pub fn to_vec<T: Copy + Default>(&self) -> Result<Vec<T>> {
        let n = self.length() / size_of::<T>();
        let mut out = vec![T::default(); n];
        // SAFETY: `out` is writable for n * size_of::<T>() bytes, which the library checks against the buffer's length.
        check(unsafe { ffi::lh_buffer_read(self.raw, 0, out.as_mut_ptr() as *mut c_void, n * size_of::<T>()) })?;
        Ok(out)
    }

    /// `MetalBuffer::copy_from_bytes(src, offset)` (buffer.rs:116-131).
    pub fn copy_from_bytes(&self, src: &[u8], offset: usize) -> Result<()> {
        // SAFETY: `src` is readable for its length; the library checks the destination range.
        check(unsafe { ffi::lh_buffer_write(self.raw, offset, src.as_ptr() as *const c_void, src.len()) })
    }

    /// Zero-fill (QuantizedKvCache::reset, quant_cache.rs:367-380).
    pub fn fill_zero(&self) -> Result<()> {
        // SAFETY: live handle.
        check(unsafe { ffi::lh_buffer_fill_zero(self.raw) })
    }

    pub fn as_ptr(&self) -> *mut ffi::lh_buffer {
        self.raw
    }
}

impl Drop for Buffer {
    fn drop(&mut self) {
        // SAFETY: created by this crate; the library defers the release while a recorded batch may still use the memory.
        unsafe { ffi::lh_buffer_free(self.raw) }
    }
}
