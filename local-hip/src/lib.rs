//! HIP (MI355X / gfx950) backend behind the kernel-dispatch API that `local-engine` calls on `local-metal`.
//!
//! * `ffi`      raw declarations of `liblocal_hip.so`, generated from `include/local_hip.h` (gen_ffi.py)
//! * `error`    `Error` / `Result` with the variants and messages of `local_metal::Error`
//! * `context`  `Context` (device + in-order stream; `MetalContext`)
//! * `buffer`   `Buffer` (device memory; `MetalBuffer`)
//! * `batch`    `CommandBatch`
//! * `kernels`  `Kernels`: one method per dispatch operation, generated from the header (gen_safe.py)
//! and, below, the host-side helpers of the TurboQuant codec that take plain slices.
//!
//! None of this has been compiled where the library is developed (no Rust toolchain there): the generated files are
//! held to the header textually by tests/test_ffi_binding.py, the hand-written ones are short and reviewed by eye.
pub mod batch;
pub mod buffer;
pub mod context;
pub mod error;
pub mod ffi;
pub mod kernels;

pub use batch::{BufferCopyRequest, CommandBatch};
pub use buffer::Buffer;
pub use context::Context;
pub use error::{last_error, Error, Result};
pub use kernels::Kernels;

/// `TurboQuant::levels` (local-engine/src/turboquant.rs:114-166): the 2^bits Lloyd-Max levels for `dim`, already divided
/// by sqrt(dim).
pub fn turboquant_levels(dim: u32, bits: u32) -> Result<Vec<f32>> {
    let mut out = vec![0.0f32; 1usize << bits];
    // SAFETY: `out` holds 2^bits floats, which is what the call writes.
    error::check(unsafe { ffi::lh_turboquant_levels(dim, bits, out.as_mut_ptr()) })?;
    Ok(out)
}

/// `Rotation::new(dim, seed).signs` (turboquant.rs:60-97): the +-1 diagonal of the randomised Hadamard rotation.
pub fn turboquant_signs(dim: u32, seed: u64) -> Result<Vec<f32>> {
    let mut out = vec![0.0f32; dim as usize];
    // SAFETY: `out` holds `dim` floats.
    error::check(unsafe { ffi::lh_turboquant_signs(dim, seed, out.as_mut_ptr()) })?;
    Ok(out)
}

/// `code_bytes(dim, bits)` (kv_cache/quant_cache.rs:30-40).
pub fn turboquant_code_bytes(dim: u32, bits: u32) -> u32 {
    // SAFETY: pure function.
    unsafe { ffi::lh_turboquant_code_bytes(dim, bits) }
}

/// `swa_ring_capacity(window, max_positions)` (quant_cache.rs:48-54).
pub fn swa_ring_capacity(window: usize, max_positions: usize) -> usize {
    // SAFETY: pure function.
    unsafe { ffi::lh_swa_ring_capacity(window, max_positions) }
}

/// `flash_split_count(eff_seq_len)` (local-metal/src/kernels.rs:1265-1278).
pub fn flash_split_count(eff_seq_len: u32) -> u32 {
    // SAFETY: pure function.
    unsafe { ffi::lh_flash_split_count(eff_seq_len) }
}

/// `lh_flash_attention_tq_rotated_lazy_into` (include/local_hip.h): the attend step of `fused_attention_into`
/// (quant_cache.rs:571-589) and, where it rides in the merge launch, the rotation back out of code space
/// (quant_cache.rs:590-598).  `Ok(true)`: `out_f16` holds the rotated heads.  `Ok(false)`: the f32 heads in `out` are still
/// in code space and the caller's output projection rotates them (`Kernels::matvec_quant_rotated_into`).
#[allow(clippy::too_many_arguments)]
pub fn flash_attention_tq_rotated_lazy_into(batch: &mut CommandBatch, rq: &Buffer, k_codes: &Buffer, k_norms: &Buffer,
                                            v_codes: &Buffer, v_norms: &Buffer, levels: &Buffer, signs: &Buffer, out: &Buffer,
                                            out_f16: &Buffer, head_dim: u32, kv_len: u32, current_pos: u32, num_q_heads: u32,
                                            num_kv_heads: u32, window: u32, bits: u32, ring_capacity: u32) -> Result<bool> {
    let mut rotated: core::ffi::c_int = 0;
    // SAFETY: every pointer comes from a live handle of this crate or from a local; the library validates sizes and shapes.
    error::check(unsafe {
        ffi::lh_flash_attention_tq_rotated_lazy_into(batch.as_ptr(), rq.as_ptr(), k_codes.as_ptr(), k_norms.as_ptr(),
                                                     v_codes.as_ptr(), v_norms.as_ptr(), levels.as_ptr(), signs.as_ptr(),
                                                     out.as_ptr(), out_f16.as_ptr(), head_dim, kv_len, current_pos,
                                                     num_q_heads, num_kv_heads, window, bits, ring_capacity, &mut rotated)
    })?;
    Ok(rotated != 0)
}
