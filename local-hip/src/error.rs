//! `Error`: the variants and `Display` strings of `local_metal::Error` (local-metal/src/error.rs:1-32), built from the
//! status code a library call returns and the message it left (`lh_last_error`).
use core::ffi::{c_int, CStr};
use core::fmt;

use crate::ffi;

#[derive(Debug)]
pub enum Error {
    /// `NoMetalDevice` / `NoDevice` of the reference: no usable HIP device (or not a gfx950 one).
    NoDevice(String),
    NoCommandQueue,
    BufferAllocation { size: usize, reason: String },
    LibraryCreation(String),
    PipelineCreation(String),
    ShaderNotFound(String),
    /// GPU-side failures surface at the wait on a batch (batch.rs:136-144), kernel-reported faults included.
    CommandBuffer(String),
    InvalidArgument(String),
    Io(std::io::Error),
}

pub type Result<T> = core::result::Result<T, Error>;

impl fmt::Display for Error {
    fn fmt(&self, f: &mut fmt::Formatter<'_>) -> fmt::Result {
        match self {
            Error::NoDevice(m) => write!(f, "No HIP device found ({m})"),
            Error::NoCommandQueue => write!(f, "Failed to create command queue"),
            Error::BufferAllocation { size, reason } => write!(f, "Buffer allocation failed (size={size}): {reason}"),
            Error::LibraryCreation(m) => write!(f, "Failed to create Metal library: {m}"),
            Error::PipelineCreation(m) => write!(f, "Failed to create pipeline state: {m}"),
            Error::ShaderNotFound(m) => write!(f, "Shader function not found: {m}"),
            Error::CommandBuffer(m) => write!(f, "Command buffer error: {m}"),
            Error::InvalidArgument(m) => write!(f, "Invalid argument: {m}"),
            Error::Io(e) => write!(f, "I/O error: {e}"),
        }
    }
}

impl std::error::Error for Error {}

impl From<std::io::Error> for Error {
    fn from(e: std::io::Error) -> Self {
        Error::Io(e)
    }
}

/// Message of the last failed call on this thread, already in the reference's wording, prefix included.
pub fn last_error() -> String {
    // SAFETY: lh_last_error returns a NUL-terminated thread-local buffer that stays valid until the next failing call
    // on this thread.
    unsafe { CStr::from_ptr(ffi::lh_last_error()) }.to_string_lossy().into_owned()
}

/// The part of a library message behind the variant's fixed prefix.
fn detail(prefix: &str) -> String {
    let full = last_error();
    full.strip_prefix(prefix).map(str::to_owned).unwrap_or(full)
}

/// Status code of a library call -> `Result`.
pub fn check(status: c_int) -> Result<()> {
    match status {
        ffi::LH_OK => Ok(()),
        ffi::LH_ERR_NO_DEVICE => Err(Error::NoDevice(last_error())),
        ffi::LH_ERR_NO_COMMAND_QUEUE => Err(Error::NoCommandQueue),
        ffi::LH_ERR_BUFFER_ALLOCATION => {
            // "Buffer allocation failed (size=N: reason)"
            let msg = last_error();
            let size = msg.split("size=").nth(1).and_then(|t| t.split(|c: char| !c.is_ascii_digit()).next())
                .and_then(|d| d.parse().ok()).unwrap_or(0);
            Err(Error::BufferAllocation { size, reason: msg })
        }
        ffi::LH_ERR_LIBRARY_CREATION => Err(Error::LibraryCreation(detail("Failed to create Metal library: "))),
        ffi::LH_ERR_PIPELINE_CREATION => Err(Error::PipelineCreation(detail("Failed to create pipeline state: "))),
        ffi::LH_ERR_SHADER_NOT_FOUND => Err(Error::ShaderNotFound(detail("Shader function not found: "))),
        ffi::LH_ERR_COMMAND_BUFFER => Err(Error::CommandBuffer(detail("Command buffer error: "))),
        ffi::LH_ERR_IO => Err(Error::Io(std::io::Error::new(std::io::ErrorKind::Other, detail("I/O error: ")))),
        _ => Err(Error::InvalidArgument(detail("Invalid argument: "))),
    }
}
