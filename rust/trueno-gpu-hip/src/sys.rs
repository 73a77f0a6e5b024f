//! Stands where `trueno-gpu/src/driver/sys.rs` stands: the same handle types and the same `CudaDriver` table of
//! function pointers (field names and signatures of sys.rs:99-201), filled from `libtrueno_hip.so`.  The rest of
//! trueno-gpu's `driver/` - context, module, stream, memory - calls through this table and needs no change.
//!
//! What differs from the CUDA table:
//! * result codes other than 0 are `hipError_t` values (`error_name` / `error_string` below name them);
//! * `cuModuleLoadData` takes a gfx950 code object (an ELF image), not PTX text.  The kernels of the k-quant path
//!   ship inside the library: `trnModuleLoadBuiltin` loads them, which is what `CudaModule::from_builtin` calls
//!   where the reference calls `CudaModule::from_ptx(&ctx, &kernel.emit_ptx())` (driver/module.rs:62-79);
//! * for the built-in k-quant kernels `cuLaunchKernel` ignores the grid, block and shared-memory arguments and
//!   uses the kernel's own geometry, so callers that pass the reference's documented `LaunchConfig` keep working.

use std::ffi::{c_char, c_int, c_uint, c_void, CStr};
use std::sync::OnceLock;

use libloading::Library;

use crate::ffi::trn_gemv_desc;

pub type CUresult = c_int;
pub type CUdevice = c_int;
pub type CUcontext = *mut c_void;
pub type CUmodule = *mut c_void;
pub type CUfunction = *mut c_void;
pub type CUstream = *mut c_void;
pub type CUdeviceptr = u64;

pub const CUDA_SUCCESS: CUresult = 0;
pub const CUDA_ERROR_INVALID_VALUE: CUresult = 1; // hipErrorInvalidValue
pub const CUDA_ERROR_OUT_OF_MEMORY: CUresult = 2; // hipErrorOutOfMemory
pub const CUDA_ERROR_NO_DEVICE: CUresult = 100; // hipErrorNoDevice
pub const CUDA_ERROR_INVALID_DEVICE: CUresult = 101; // hipErrorInvalidDevice
pub const CUDA_ERROR_NOT_FOUND: CUresult = 500; // hipErrorNotFound
pub const CUDA_ERROR_LAUNCH_FAILED: CUresult = 719; // hipErrorLaunchFailure

/// The driver table.  The first 25 fields are those of the reference's `CudaDriver`; the `trn*` fields have no
/// counterpart there.
pub struct CudaDriver {
    pub cuInit: unsafe extern "C" fn(flags: c_uint) -> CUresult,
    pub cuDeviceGetCount: unsafe extern "C" fn(count: *mut c_int) -> CUresult,
    pub cuDeviceGet: unsafe extern "C" fn(device: *mut CUdevice, ordinal: c_int) -> CUresult,
    pub cuDeviceGetName: unsafe extern "C" fn(name: *mut c_char, len: c_int, device: CUdevice) -> CUresult,
    pub cuDeviceTotalMem: unsafe extern "C" fn(bytes: *mut usize, device: CUdevice) -> CUresult,
    pub cuDevicePrimaryCtxRetain: unsafe extern "C" fn(ctx: *mut CUcontext, device: CUdevice) -> CUresult,
    pub cuDevicePrimaryCtxRelease: unsafe extern "C" fn(device: CUdevice) -> CUresult,
    pub cuCtxSetCurrent: unsafe extern "C" fn(ctx: CUcontext) -> CUresult,
    pub cuCtxSynchronize: unsafe extern "C" fn() -> CUresult,
    pub cuModuleLoadData: unsafe extern "C" fn(module: *mut CUmodule, image: *const c_void) -> CUresult,
    pub cuModuleUnload: unsafe extern "C" fn(module: CUmodule) -> CUresult,
    pub cuModuleGetFunction:
        unsafe extern "C" fn(func: *mut CUfunction, module: CUmodule, name: *const c_char) -> CUresult,
    pub cuMemAlloc: unsafe extern "C" fn(ptr: *mut CUdeviceptr, size: usize) -> CUresult,
    pub cuMemFree: unsafe extern "C" fn(ptr: CUdeviceptr) -> CUresult,
    pub cuMemcpyHtoD: unsafe extern "C" fn(dst: CUdeviceptr, src: *const c_void, size: usize) -> CUresult,
    pub cuMemcpyDtoH: unsafe extern "C" fn(dst: *mut c_void, src: CUdeviceptr, size: usize) -> CUresult,
    pub cuMemcpyHtoDAsync:
        unsafe extern "C" fn(dst: CUdeviceptr, src: *const c_void, size: usize, stream: CUstream) -> CUresult,
    pub cuMemcpyDtoHAsync:
        unsafe extern "C" fn(dst: *mut c_void, src: CUdeviceptr, size: usize, stream: CUstream) -> CUresult,
    pub cuMemcpyDtoD: unsafe extern "C" fn(dst: CUdeviceptr, src: CUdeviceptr, size: usize) -> CUresult,
    pub cuMemcpyDtoDAsync:
        unsafe extern "C" fn(dst: CUdeviceptr, src: CUdeviceptr, size: usize, stream: CUstream) -> CUresult,
    pub cuMemGetInfo: unsafe extern "C" fn(free: *mut usize, total: *mut usize) -> CUresult,
    pub cuStreamCreate: unsafe extern "C" fn(stream: *mut CUstream, flags: c_uint) -> CUresult,
    pub cuStreamDestroy: unsafe extern "C" fn(stream: CUstream) -> CUresult,
    pub cuStreamSynchronize: unsafe extern "C" fn(stream: CUstream) -> CUresult,
    #[allow(clippy::type_complexity)]
    pub cuLaunchKernel: unsafe extern "C" fn(
        func: CUfunction,
        grid_dim_x: c_uint,
        grid_dim_y: c_uint,
        grid_dim_z: c_uint,
        block_dim_x: c_uint,
        block_dim_y: c_uint,
        block_dim_z: c_uint,
        shared_mem_bytes: c_uint,
        stream: CUstream,
        kernel_params: *mut *mut c_void,
        extra: *mut *mut c_void,
    ) -> CUresult,

    /// `trn_module_load_builtin`: the gfx950 code object that ships inside the library.
    pub trnModuleLoadBuiltin: unsafe extern "C" fn(module: *mut CUmodule) -> CUresult,
    /// `trn_kquant_gemv_batch`: a decode step's GEMVs as one list; independent neighbours share a launch.
    pub trnKquantGemvBatch: unsafe extern "C" fn(stream: CUstream, descs: *const trn_gemv_desc, count: u32) -> CUresult,
    /// `trn_function_set_rmsnorm`, `trn_function_set_attention`: what the reference compiles into the PTX of one
    /// kernel instance, set on the function handle before a by-name launch of `rmsnorm`, `fused_residual_rmsnorm`
    /// or `incremental_attention`.
    pub trnFunctionSetRmsnorm: unsafe extern "C" fn(func: CUfunction, hidden_size: u32, epsilon: f32) -> CUresult,
    #[allow(clippy::type_complexity)]
    pub trnFunctionSetAttention: unsafe extern "C" fn(
        func: CUfunction,
        head_dim: u32,
        num_heads: u32,
        num_kv_heads: u32,
        max_seq_len: u32,
        scale: f32,
    ) -> CUresult,
    pub trnErrorName: unsafe extern "C" fn(status: CUresult) -> *const c_char,
    pub trnErrorString: unsafe extern "C" fn(status: CUresult) -> *const c_char,
}

static LIBRARY: OnceLock<Option<Library>> = OnceLock::new();
static DRIVER: OnceLock<Option<CudaDriver>> = OnceLock::new();

/// Where the library is looked for: `TRN_HIP_LIBRARY` if set, then the loader's search path.
fn library_names() -> Vec<String> {
    let mut names = Vec::new();
    if let Ok(path) = std::env::var("TRN_HIP_LIBRARY") {
        names.push(path);
    }
    names.push("libtrueno_hip.so".to_string());
    names
}

impl CudaDriver {
    /// The table, loaded once.  `None` when the library is not there - like the reference's `load()` on a machine
    /// without a CUDA driver, not an error by itself.
    #[must_use]
    pub fn load() -> Option<&'static Self> {
        let library = LIBRARY.get_or_init(|| {
            // SAFETY: loading this library runs no code of ours beyond its static initialisers
            library_names().iter().find_map(|name| unsafe { Library::new(name) }.ok())
        });
        DRIVER.get_or_init(|| Self::from_library(library.as_ref()?)).as_ref()
    }

    fn from_library(lib: &Library) -> Option<Self> {
        macro_rules! sym {
            ($name:literal) => {{
                // SAFETY: the symbol has the C signature of the field it is assigned to (include/trueno_hip.h)
                let symbol = unsafe { lib.get($name) }.ok()?;
                *symbol
            }};
        }
        Some(Self {
            cuInit: sym!(b"trn_init\0"),
            cuDeviceGetCount: sym!(b"trn_device_get_count\0"),
            cuDeviceGet: sym!(b"trn_device_get\0"),
            cuDeviceGetName: sym!(b"trn_device_get_name\0"),
            cuDeviceTotalMem: sym!(b"trn_device_total_mem\0"),
            cuDevicePrimaryCtxRetain: sym!(b"trn_primary_ctx_retain\0"),
            cuDevicePrimaryCtxRelease: sym!(b"trn_primary_ctx_release\0"),
            cuCtxSetCurrent: sym!(b"trn_ctx_set_current\0"),
            cuCtxSynchronize: sym!(b"trn_ctx_synchronize\0"),
            cuModuleLoadData: sym!(b"trn_module_load_data\0"),
            cuModuleUnload: sym!(b"trn_module_unload\0"),
            cuModuleGetFunction: sym!(b"trn_module_get_function\0"),
            cuMemAlloc: sym!(b"trn_mem_alloc\0"),
            cuMemFree: sym!(b"trn_mem_free\0"),
            cuMemcpyHtoD: sym!(b"trn_memcpy_htod\0"),
            cuMemcpyDtoH: sym!(b"trn_memcpy_dtoh\0"),
            cuMemcpyHtoDAsync: sym!(b"trn_memcpy_htod_async\0"),
            cuMemcpyDtoHAsync: sym!(b"trn_memcpy_dtoh_async\0"),
            cuMemcpyDtoD: sym!(b"trn_memcpy_dtod\0"),
            cuMemcpyDtoDAsync: sym!(b"trn_memcpy_dtod_async\0"),
            cuMemGetInfo: sym!(b"trn_mem_get_info\0"),
            cuStreamCreate: sym!(b"trn_stream_create\0"),
            cuStreamDestroy: sym!(b"trn_stream_destroy\0"),
            cuStreamSynchronize: sym!(b"trn_stream_synchronize\0"),
            cuLaunchKernel: sym!(b"trn_launch_kernel\0"),
            trnModuleLoadBuiltin: sym!(b"trn_module_load_builtin\0"),
            trnKquantGemvBatch: sym!(b"trn_kquant_gemv_batch\0"),
            trnFunctionSetRmsnorm: sym!(b"trn_function_set_rmsnorm\0"),
            trnFunctionSetAttention: sym!(b"trn_function_set_attention\0"),
            trnErrorName: sym!(b"trn_error_name\0"),
            trnErrorString: sym!(b"trn_error_string\0"),
        })
    }

    /// `Ok(())` for 0, otherwise the code with its name and description (the reference's `check` wraps the same
    /// pair into `GpuError::CudaDriver(String, i32)`, sys.rs:355-365).
    pub fn check(result: CUresult) -> Result<(), (String, CUresult)> {
        if result == CUDA_SUCCESS {
            Ok(())
        } else {
            Err((error_string(result), result))
        }
    }
}

/// "hipErrorInvalidValue: invalid argument" for 1, and so on; the code alone when the library is not loaded.
#[must_use]
pub fn error_string(result: CUresult) -> String {
    let Some(driver) = CudaDriver::load() else {
        return format!("error {result}");
    };
    // SAFETY: both functions return pointers to static NUL-terminated strings
    let (name, text) = unsafe { (CStr::from_ptr((driver.trnErrorName)(result)), CStr::from_ptr((driver.trnErrorString)(result))) };
    format!("{}: {}", name.to_string_lossy(), text.to_string_lossy())
}
