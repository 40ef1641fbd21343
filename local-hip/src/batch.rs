//! `CommandBatch`: the dispatches of one step on the context's in-order stream, behind the method names of
//! `local_metal::CommandBatch` (local-metal/src/batch.rs:147-291).  Metal encodes into a command buffer and runs it at
//! commit; here a dispatch starts as soon as it is encoded and `commit_and_wait` is the wait.
use core::ptr;

use crate::buffer::Buffer;
use crate::context::Context;
use crate::error::{check, Result};
use crate::ffi;

pub struct CommandBatch {
    raw: *mut ffi::lh_batch,
}

unsafe impl Send for CommandBatch {}

/// One device-to-device copy of `blit_buffer_copies` (batch.rs:33-44 `BufferCopyRequest`).
pub struct BufferCopyRequest<'a> {
    pub src: &'a Buffer,
    pub src_offset: usize,
    pub dst: &'a Buffer,
    pub dst_offset: usize,
    pub len: usize,
}

impl CommandBatch {
    /// `CommandBatch::new(ctx)` (batch.rs:154).
    pub fn new(ctx: &Context) -> Result<Self> {
        let mut raw = ptr::null_mut();
        // SAFETY: valid out pointer.
        check(unsafe { ffi::lh_batch_new(ctx.as_ptr(), &mut raw) })?;
        Ok(CommandBatch { raw })
    }

    /// `dispatch_count()` (batch.rs:174-182).
    pub fn dispatch_count(&self) -> u32 {
        // SAFETY: live handle.
        unsafe { ffi::lh_batch_dispatch_count(self.raw) }
    }

    /// `blit_buffer_copies(copies)` (batch.rs:200-238): out-of-range requests are refused before anything is enqueued.
    pub fn blit_buffer_copies<'a, I: IntoIterator<Item = BufferCopyRequest<'a>>>(&mut self, copies: I) -> Result<()> {
        for c in copies {
            // SAFETY: live handles; the library checks both ranges.
            check(unsafe { ffi::lh_batch_blit_copy(self.raw, c.src.as_ptr(), c.src_offset, c.dst.as_ptr(), c.dst_offset, c.len) })?;
        }
        Ok(())
    }

    /// `commit_and_wait()` (batch.rs:240-250).  The reference consumes the batch; this one stays usable, which is what
    /// `commit_and_renew` gives there.
    pub fn commit_and_wait(&mut self) -> Result<()> {
        // SAFETY: live handle.
        check(unsafe { ffi::lh_batch_commit_and_wait(self.raw) })
    }

    /// `submit_and_renew(ctx)` (batch.rs:252-267): nothing to flush, work runs as it is encoded.
    pub fn submit_and_renew(&mut self, _ctx: &Context) -> Result<()> {
        // SAFETY: live handle.
        check(unsafe { ffi::lh_batch_submit_and_renew(self.raw) })
    }

    /// `commit_and_renew(ctx)` (batch.rs:269-280).
    pub fn commit_and_renew(&mut self, _ctx: &Context) -> Result<()> {
        // SAFETY: live handle.
        check(unsafe { ffi::lh_batch_commit_and_renew(self.raw) })
    }

    pub fn as_ptr(&self) -> *mut ffi::lh_batch {
        self.raw
    }
}

impl Drop for CommandBatch {
    fn drop(&mut self) {
        // SAFETY: created by lh_batch_new.
        unsafe { ffi::lh_batch_free(self.raw) }
    }
}
