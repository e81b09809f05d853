//! `ojas_core::Backend` for AMD MI355X (gfx950).
//!
//! The device side is `libojas_mi355x.so`: hand-written HIP kernels behind the C ABI of
//! `include/ojas_mi355x.h`. This crate is the host side and holds no arithmetic: every trait
//! method runs its `ojas_core::shapes` validator, checks placement, reserves the output from the
//! budget and calls one entry point. It implements the GPT op set (linear / gemm, causal SDPA,
//! RMSNorm, cross-entropy and its fusion with the head, embedding, AdamW and Muon-NS5, clip) plus
//! the ops of the nanolab block and of decoding; every other method keeps the trait's default,
//! which refuses by name (`unsupported_op`, ojas-core/src/backend.rs:792-797).
//!
//! Non-finite values are detected on the device and reported late, as `WgpuBackend` documents for
//! itself: an op returns `Ok`, and the next `sync`, `download` or `clip_grad_norm` returns
//! `OjasError::NonFinite` naming the first op that produced one.

pub mod backend;
pub mod buffer;
pub mod ffi;

pub use backend::Mi355xBackend;
pub use buffer::{Ctx, HipDeviceBuffer};
