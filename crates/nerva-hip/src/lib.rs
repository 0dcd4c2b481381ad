//! HIP backend boundary (MI355X, gfx950): the twin of `nerva-cuda` for the batch-1 decode session.
//!
//! Rust owns the public capability surface; libnerva_hip owns the HIP runtime calls and the kernels.
//! `ffi` is generated from the library's C header, `session` holds the safe wrappers with the names
//! and error behaviour of nerva-cuda's (`Cuda` -> `Hip`), `contracts` names the kernel-contract rows
//! this backend registers.

pub mod contracts;
pub mod ffi;
pub mod session;

#[cfg(nerva_hip_native_stubs)]
mod native_stubs;
