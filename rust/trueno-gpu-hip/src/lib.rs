//! Binding of trueno-gpu's driver layer and k-quant kernels to `libtrueno_hip.so` (MI355X, gfx950).
//!
//! `sys` is the replacement for `trueno-gpu/src/driver/sys.rs`; `ffi` the whole C ABI of `include/trueno_hip.h`;
//! `kernels` the k-quant kernel types of `trueno-gpu/src/kernels/quantize.rs` on top of it.

#![allow(non_snake_case, non_camel_case_types, clippy::missing_safety_doc, clippy::too_many_arguments)]

pub mod ffi;
/// The typed launchers call the library's entry points directly: with the `link` feature only.
#[cfg(feature = "link")]
pub mod kernels;
pub mod sys;

pub use ffi::{trn_gemv_desc, TRN_GEMV_NORM_INPUT, TRN_GEMV_SWIGLU_INPUT};
pub use sys::{CUcontext, CUdevice, CUdeviceptr, CUfunction, CUmodule, CUresult, CUstream, CudaDriver};
