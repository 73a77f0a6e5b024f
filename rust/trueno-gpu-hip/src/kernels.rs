//! The k-quant kernel types of `trueno-gpu/src/kernels/quantize.rs`, on top of the C ABI: the same constructors,
//! field names, `name()` strings and kernel parameter order.  `build_ptx` / `emit_ptx` / `as_module`
//! (kernels/mod.rs:47-102) have no meaning without a PTX back end: a kernel here is launched by its typed launcher
//! (`launch`) or by name from the built-in module with the reference's parameter list (`kernel_params`).

use crate::ffi;
use crate::sys::{CUdeviceptr, CUresult, CUstream, CudaDriver};

// quantize.rs:34-53
pub const Q4K_BLOCK_SIZE: u32 = 32;
pub const Q4K_SUPER_BLOCK_SIZE: u32 = 256;
pub const Q4K_SUPER_BLOCK_BYTES: u32 = 144;
pub const Q4K_BLOCK_BYTES: u32 = 18;
pub const Q5K_SUPER_BLOCK_SIZE: u32 = 256;
pub const Q5K_SUPER_BLOCK_BYTES: u32 = 176;
pub const Q6K_SUPER_BLOCK_SIZE: u32 = 256;
pub const Q6K_SUPER_BLOCK_BYTES: u32 = 210;

/// quantize.rs:56-62
#[derive(Debug, Clone, Copy, PartialEq, Eq)]
pub enum Q4KFormat {
    Simplified,
    GgmlSuperBlock,
}

/// What survives of the `Kernel` trait without PTX.
pub trait Kernel {
    /// The name under which the built-in module exports the kernel (the reference's name).
    fn name(&self) -> &str;
    /// Bytes of the quantized weight operand.
    fn weight_bytes(&self) -> u64;
}

fn check(result: CUresult) -> Result<(), (String, CUresult)> {
    CudaDriver::check(result)
}

macro_rules! gemv_kernel {
    ($type:ident, $name:literal, $bytes:expr, $launcher:path, $doc:literal) => {
        #[doc = $doc]
        #[derive(Debug, Clone)]
        pub struct $type {
            /// columns of W = length of x (a multiple of 256)
            pub k: u32,
            /// rows of W = length of y
            pub n: u32,
        }

        impl $type {
            /// `k` first, then `n`, as in the reference.
            #[must_use]
            pub fn new(k: u32, n: u32) -> Self {
                Self { k, n }
            }

            #[must_use]
            pub const fn num_super_blocks_per_row(&self) -> u32 {
                self.k / 256
            }

            /// `(y_ptr, w_ptr, x_ptr, k_dim, n_dim)`: host copies of the parameters for a launch by name.
            #[must_use]
            pub fn kernel_params(&self, y: CUdeviceptr, w: CUdeviceptr, x: CUdeviceptr) -> (CUdeviceptr, CUdeviceptr, CUdeviceptr, u32, u32) {
                (y, w, x, self.k, self.n)
            }

            /// y[n] = W[n][k] x[k] on `stream` (null: the default stream).
            ///
            /// # Safety
            /// `y`, `w`, `x` must be device addresses of at least `n` floats, `weight_bytes()` bytes and `k` floats.
            pub unsafe fn launch(&self, stream: CUstream, y: CUdeviceptr, w: CUdeviceptr, x: CUdeviceptr) -> Result<(), (String, CUresult)> {
                check($launcher(stream, y, w, x, self.k, self.n))
            }
        }

        impl Kernel for $type {
            fn name(&self) -> &str {
                $name
            }
            fn weight_bytes(&self) -> u64 {
                u64::from(self.n) * u64::from(self.num_super_blocks_per_row()) * u64::from($bytes)
            }
        }
    };
}

gemv_kernel!(Q4KGemvKernel, "q4k_gemv_warp_reduce", Q4K_SUPER_BLOCK_BYTES, ffi::trn_q4k_gemv, "quantize.rs:1157-1523");
gemv_kernel!(Q5KGemvKernel, "q5k_gemv_warp_reduce", Q5K_SUPER_BLOCK_BYTES, ffi::trn_q5k_gemv, "quantize.rs:1532-1720");
gemv_kernel!(Q6KGemvKernel, "q6k_gemv_warp_reduce", Q6K_SUPER_BLOCK_BYTES, ffi::trn_q6k_gemv, "quantize.rs:1733-1940");

macro_rules! gemm_kernel {
    ($type:ident, $name:literal, $bytes:expr, $launcher:path, $as_written:path, $doc:literal) => {
        #[doc = $doc]
        #[derive(Debug, Clone)]
        pub struct $type {
            pub m: u32,
            pub n: u32,
            pub k: u32,
            pub tile_size: u32,
        }

        impl $type {
            #[must_use]
            pub fn new(m: u32, n: u32, k: u32) -> Self {
                Self { m, n, k, tile_size: 32 }
            }

            #[must_use]
            pub const fn with_tile_size(mut self, tile_size: u32) -> Self {
                self.tile_size = tile_size;
                self
            }

            #[must_use]
            pub const fn num_super_blocks_per_row(&self) -> u32 {
                self.k / 256
            }

            /// C[m][n] = A[m][k] W[n][k]^T with the canonical (GGML) decode of the weights.
            ///
            /// # Safety
            /// `a`, `b_quant`, `c` must be device addresses of `m * k` floats, `weight_bytes()` bytes and `m * n` floats.
            pub unsafe fn launch(&self, stream: CUstream, a: CUdeviceptr, b_quant: CUdeviceptr, c: CUdeviceptr) -> Result<(), (String, CUresult)> {
                check($launcher(stream, a, b_quant, c, self.m, self.n, self.k))
            }

            /// The same product with the weights decoded exactly as the reference's GEMM builder writes it.
            ///
            /// # Safety
            /// As for `launch`.
            pub unsafe fn launch_as_written(&self, stream: CUstream, a: CUdeviceptr, b_quant: CUdeviceptr, c: CUdeviceptr) -> Result<(), (String, CUresult)> {
                check($as_written(stream, a, b_quant, c, self.m, self.n, self.k))
            }
        }

        impl Kernel for $type {
            fn name(&self) -> &str {
                $name
            }
            fn weight_bytes(&self) -> u64 {
                u64::from(self.n) * u64::from(self.num_super_blocks_per_row()) * u64::from($bytes)
            }
        }
    };
}

gemm_kernel!(Q5KKernel, "q5k_gemm_ggml", Q5K_SUPER_BLOCK_BYTES, ffi::trn_q5k_gemm, ffi::trn_q5k_gemm_as_written, "quantize.rs:598-866");
gemm_kernel!(Q6KKernel, "q6k_gemm_ggml", Q6K_SUPER_BLOCK_BYTES, ffi::trn_q6k_gemm, ffi::trn_q6k_gemm_as_written, "quantize.rs:884-1121");

/// quantize.rs:66-147.  `QuantizeKernel::ggml(m, n, k)` is the 144-byte super-block format (`q4k_gemm_ggml`); the
/// plain constructor the legacy format of 18-byte blocks of 32 values (`q4k_gemm_fused`).
#[derive(Debug, Clone)]
pub struct QuantizeKernel {
    pub m: u32,
    pub n: u32,
    pub k: u32,
    pub tile_size: u32,
    pub block_size: u32,
    pub format: Q4KFormat,
}

impl QuantizeKernel {
    #[must_use]
    pub fn new(m: u32, n: u32, k: u32) -> Self {
        Self { m, n, k, tile_size: 32, block_size: Q4K_BLOCK_SIZE, format: Q4KFormat::Simplified }
    }

    #[must_use]
    pub fn ggml(m: u32, n: u32, k: u32) -> Self {
        Self { m, n, k, tile_size: 32, block_size: Q4K_SUPER_BLOCK_SIZE, format: Q4KFormat::GgmlSuperBlock }
    }

    #[must_use]
    pub const fn with_tile_size(mut self, tile_size: u32) -> Self {
        self.tile_size = tile_size;
        self
    }

    #[must_use]
    pub const fn num_blocks_per_row(&self) -> u32 {
        self.k / self.block_size
    }

    #[must_use]
    pub const fn num_super_blocks_per_row(&self) -> u32 {
        self.k / Q4K_SUPER_BLOCK_SIZE
    }

    /// C[m][n] = A[m][k] W[n][k]^T.
    ///
    /// # Safety
    /// `a`, `b_quant`, `c` must be device addresses of `m * k` floats, `weight_bytes()` bytes and `m * n` floats.
    pub unsafe fn launch(&self, stream: CUstream, a: CUdeviceptr, b_quant: CUdeviceptr, c: CUdeviceptr) -> Result<(), (String, CUresult)> {
        check(match self.format {
            Q4KFormat::GgmlSuperBlock => ffi::trn_q4k_gemm(stream, a, b_quant, c, self.m, self.n, self.k),
            Q4KFormat::Simplified => ffi::trn_q4k_gemm_fused(stream, a, b_quant, c, self.m, self.n, self.k),
        })
    }
}

impl Kernel for QuantizeKernel {
    fn name(&self) -> &str {
        match self.format {
            Q4KFormat::GgmlSuperBlock => "q4k_gemm_ggml",
            Q4KFormat::Simplified => "q4k_gemm_fused",
        }
    }
    fn weight_bytes(&self) -> u64 {
        match self.format {
            Q4KFormat::GgmlSuperBlock => u64::from(self.n) * u64::from(self.num_super_blocks_per_row()) * u64::from(Q4K_SUPER_BLOCK_BYTES),
            Q4KFormat::Simplified => u64::from(self.n) * u64::from(self.num_blocks_per_row()) * u64::from(Q4K_BLOCK_BYTES),
        }
    }
}

/// A decode step's GEMVs as one list: the library finds the entries that do not depend on one another from their
/// pointer ranges and puts them into one launch (`trn_kquant_gemv_batch`).  No counterpart in the reference, which
/// launches one kernel per GEMV.
#[derive(Debug, Default, Clone)]
pub struct GemvBatch {
    pub descs: Vec<ffi::trn_gemv_desc>,
}

impl GemvBatch {
    #[must_use]
    pub fn new() -> Self {
        Self::default()
    }

    /// y = W x for a matrix of format `fmt` (4, 5 or 6: Q4_K, Q5_K, Q6_K).
    pub fn add(&mut self, fmt: u32, k: u32, n: u32, y: CUdeviceptr, w: CUdeviceptr, x: CUdeviceptr) -> &mut Self {
        self.descs.push(ffi::trn_gemv_desc { fmt, k, n, y, w, x, ..Default::default() });
        self
    }

    /// Issues the list on `stream`.
    ///
    /// # Safety
    /// Every entry's addresses must be valid for its shape.
    pub unsafe fn launch(&self, stream: CUstream) -> Result<(), (String, CUresult)> {
        check(ffi::trn_kquant_gemv_batch(stream, self.descs.as_ptr(), self.descs.len() as u32))
    }
}
