//! `extern "C"` declarations of every entry point of `include/trueno_hip.h`, in the header's order.
//! Handles are opaque pointers; `trn_dptr` is a device address; `trn_status` is 0 on success and a `hipError_t`
//! value (or one of the library's own two codes) otherwise.

use std::ffi::{c_char, c_int, c_uint, c_void};

pub type trn_status = c_int;
pub type trn_device = c_int;
pub type trn_ctx = *mut c_void;
pub type trn_module = *mut c_void;
pub type trn_function = *mut c_void;
pub type trn_stream = *mut c_void;
pub type trn_dptr = u64;
pub type trn_event = *mut c_void;

pub const TRN_SUCCESS: trn_status = 0;
pub const TRN_ERROR_INVALID_VALUE: trn_status = 1;
pub const TRN_ERROR_NO_DEVICE: trn_status = 100;
pub const TRN_ERROR_INVALID_DEVICE: trn_status = 101;
pub const TRN_ERROR_NOT_FOUND: trn_status = 500;
/// A device-side wait of the one-launch executor ran out of its budget; the results of that list are not valid.
pub const TRN_ERROR_WAIT_ABANDONED: trn_status = 9001;
/// `trn_q4k_gemm_noalloc`: the product needs more scratch memory than the library's static buffer holds.
pub const TRN_ERROR_SCRATCH_TOO_SMALL: trn_status = 9002;
pub const TRN_STREAM_NON_BLOCKING: c_uint = 1;

pub const TRN_GEMV_NORM_INPUT: u32 = 1;
pub const TRN_GEMV_SWIGLU_INPUT: u32 = 8;

/// One entry of a GEMV list (`trn_kquant_gemv_batch`).  `fmt` is 4, 5 or 6 (Q4_K, Q5_K, Q6_K); the last five fields
/// are zero for a plain `y = W x`.
#[repr(C)]
#[derive(Clone, Copy, Debug, Default)]
pub struct trn_gemv_desc {
    pub fmt: u32,
    pub k: u32,
    pub n: u32,
    pub flags: u32,
    pub y: trn_dptr,
    pub w: trn_dptr,
    pub x: trn_dptr,
    pub gamma: trn_dptr,
    pub x2: trn_dptr,
    pub residual: trn_dptr,
    pub norm_eps: f32,
    pub reserved: u32,
}

#[cfg_attr(feature = "link", link(name = "trueno_hip"))]
extern "C" {
    // 1. initialisation, 2. devices, 3. contexts
    pub fn trn_init(flags: c_uint) -> trn_status;
    pub fn trn_device_get_count(count: *mut c_int) -> trn_status;
    pub fn trn_device_get(device: *mut trn_device, ordinal: c_int) -> trn_status;
    pub fn trn_device_get_name(name: *mut c_char, len: c_int, device: trn_device) -> trn_status;
    pub fn trn_device_total_mem(bytes: *mut usize, device: trn_device) -> trn_status;
    pub fn trn_primary_ctx_retain(ctx: *mut trn_ctx, device: trn_device) -> trn_status;
    pub fn trn_primary_ctx_release(device: trn_device) -> trn_status;
    pub fn trn_ctx_set_current(ctx: trn_ctx) -> trn_status;
    pub fn trn_ctx_synchronize() -> trn_status;

    // 4. modules
    pub fn trn_module_load_data(module: *mut trn_module, image: *const c_void) -> trn_status;
    pub fn trn_module_unload(module: trn_module) -> trn_status;
    pub fn trn_module_get_function(func: *mut trn_function, module: trn_module, name: *const c_char) -> trn_status;
    pub fn trn_function_set_rmsnorm(func: trn_function, hidden_size: u32, epsilon: f32) -> trn_status;
    pub fn trn_function_set_attention(
        func: trn_function,
        head_dim: u32,
        num_heads: u32,
        num_kv_heads: u32,
        max_seq_len: u32,
        scale: f32,
    ) -> trn_status;

    // 5. memory
    pub fn trn_mem_alloc(ptr: *mut trn_dptr, size: usize) -> trn_status;
    pub fn trn_mem_free(ptr: trn_dptr) -> trn_status;
    pub fn trn_memcpy_htod(dst: trn_dptr, src: *const c_void, size: usize) -> trn_status;
    pub fn trn_memcpy_dtoh(dst: *mut c_void, src: trn_dptr, size: usize) -> trn_status;
    pub fn trn_memcpy_htod_async(dst: trn_dptr, src: *const c_void, size: usize, stream: trn_stream) -> trn_status;
    pub fn trn_memcpy_dtoh_async(dst: *mut c_void, src: trn_dptr, size: usize, stream: trn_stream) -> trn_status;
    pub fn trn_memcpy_dtod(dst: trn_dptr, src: trn_dptr, size: usize) -> trn_status;
    pub fn trn_memcpy_dtod_async(dst: trn_dptr, src: trn_dptr, size: usize, stream: trn_stream) -> trn_status;
    pub fn trn_mem_get_info(free_bytes: *mut usize, total_bytes: *mut usize) -> trn_status;

    // 6. streams and launches
    pub fn trn_stream_create(stream: *mut trn_stream, flags: c_uint) -> trn_status;
    pub fn trn_stream_destroy(stream: trn_stream) -> trn_status;
    pub fn trn_stream_synchronize(stream: trn_stream) -> trn_status;
    pub fn trn_launch_kernel(
        func: trn_function,
        grid_x: c_uint,
        grid_y: c_uint,
        grid_z: c_uint,
        block_x: c_uint,
        block_y: c_uint,
        block_z: c_uint,
        shared_mem_bytes: c_uint,
        stream: trn_stream,
        kernel_params: *mut *mut c_void,
        extra: *mut *mut c_void,
    ) -> trn_status;

    // 7. the built-in code object
    pub fn trn_module_load_builtin(module: *mut trn_module) -> trn_status;
    pub fn trn_builtin_image(image: *mut *const c_void, size: *mut usize) -> trn_status;

    // 8. typed launchers of the k-quant path
    pub fn trn_q4k_gemv(stream: trn_stream, y: trn_dptr, w: trn_dptr, x: trn_dptr, k: u32, n: u32) -> trn_status;
    pub fn trn_q5k_gemv(stream: trn_stream, y: trn_dptr, w: trn_dptr, x: trn_dptr, k: u32, n: u32) -> trn_status;
    pub fn trn_q6k_gemv(stream: trn_stream, y: trn_dptr, w: trn_dptr, x: trn_dptr, k: u32, n: u32) -> trn_status;
    pub fn trn_q4k_gemm(stream: trn_stream, a: trn_dptr, b_quant: trn_dptr, c: trn_dptr, m: u32, n: u32, k: u32) -> trn_status;
    pub fn trn_q5k_gemm(stream: trn_stream, a: trn_dptr, b_quant: trn_dptr, c: trn_dptr, m: u32, n: u32, k: u32) -> trn_status;
    pub fn trn_q6k_gemm(stream: trn_stream, a: trn_dptr, b_quant: trn_dptr, c: trn_dptr, m: u32, n: u32, k: u32) -> trn_status;
    pub fn trn_q4k_gemm_noalloc(stream: trn_stream, a: trn_dptr, b_quant: trn_dptr, c: trn_dptr, m: u32, n: u32, k: u32) -> trn_status;
    pub fn trn_q4k_gemm_as_written(stream: trn_stream, a: trn_dptr, b_quant: trn_dptr, c: trn_dptr, m: u32, n: u32, k: u32) -> trn_status;
    pub fn trn_q5k_gemm_as_written(stream: trn_stream, a: trn_dptr, b_quant: trn_dptr, c: trn_dptr, m: u32, n: u32, k: u32) -> trn_status;
    pub fn trn_q6k_gemm_as_written(stream: trn_stream, a: trn_dptr, b_quant: trn_dptr, c: trn_dptr, m: u32, n: u32, k: u32) -> trn_status;
    pub fn trn_q4k_gemm_fused(stream: trn_stream, a: trn_dptr, b_quant: trn_dptr, c: trn_dptr, m: u32, n: u32, k: u32) -> trn_status;
    pub fn trn_kquant_gemv_batch(stream: trn_stream, descs: *const trn_gemv_desc, count: u32) -> trn_status;
    pub fn trn_kquant_gemv_plan(descs: *const trn_gemv_desc, count: u32, launch_of: *mut u32) -> trn_status;

    // 9. test surface: dequantise to f32
    pub fn trn_q4k_dequant_f32(stream: trn_stream, out: trn_dptr, w: trn_dptr, n_sb: u64, policy: c_int) -> trn_status;
    pub fn trn_q5k_dequant_f32(stream: trn_stream, out: trn_dptr, w: trn_dptr, n_sb: u64, policy: c_int) -> trn_status;
    pub fn trn_q6k_dequant_f32(stream: trn_stream, out: trn_dptr, w: trn_dptr, n_sb: u64, policy: c_int) -> trn_status;
    pub fn trn_q4k_simplified_dequant_f32(stream: trn_stream, out: trn_dptr, w: trn_dptr, n_blocks: u64) -> trn_status;

    // 10. timing, errors, tuning; the neighbours of the path
    pub fn trn_event_create(event: *mut trn_event) -> trn_status;
    pub fn trn_event_destroy(event: trn_event) -> trn_status;
    pub fn trn_event_record(event: trn_event, stream: trn_stream) -> trn_status;
    pub fn trn_event_synchronize(event: trn_event) -> trn_status;
    pub fn trn_event_elapsed_ms(ms: *mut f32, start: trn_event, stop: trn_event) -> trn_status;
    pub fn trn_incremental_attention(
        stream: trn_stream,
        q: trn_dptr,
        k: trn_dptr,
        v: trn_dptr,
        out: trn_dptr,
        seq_len: u32,
        head_dim: u32,
        num_heads: u32,
        num_kv_heads: u32,
        max_seq_len: u32,
        scale: f32,
    ) -> trn_status;
    pub fn trn_q5k_from_ggml(stream: trn_stream, dst: trn_dptr, src: trn_dptr, n_sb: u64) -> trn_status;
    pub fn trn_gemv_f32(stream: trn_stream, y: trn_dptr, a: trn_dptr, x: trn_dptr, k: u32, n: u32) -> trn_status;
    pub fn trn_residual_add(stream: trn_stream, input1: trn_dptr, input2: trn_dptr, output: trn_dptr, n: u32) -> trn_status;
    pub fn trn_fused_swiglu(stream: trn_stream, gate: trn_dptr, up: trn_dptr, output: trn_dptr, n: u32) -> trn_status;
    pub fn trn_rmsnorm(stream: trn_stream, input: trn_dptr, output: trn_dptr, gamma: trn_dptr, hidden_size: u32, epsilon: f32) -> trn_status;
    pub fn trn_fused_residual_rmsnorm(
        stream: trn_stream,
        residual: trn_dptr,
        input: trn_dptr,
        output: trn_dptr,
        gamma: trn_dptr,
        hidden_size: u32,
        epsilon: f32,
    ) -> trn_status;
    pub fn trn_copy_u128(stream: trn_stream, dst: trn_dptr, src: trn_dptr, bytes: u64) -> trn_status;
    pub fn trn_read_u128(stream: trn_stream, src: trn_dptr, bytes: u64, sink: trn_dptr) -> trn_status;
    pub fn trn_error_name(status: trn_status) -> *const c_char;
    pub fn trn_error_string(status: trn_status) -> *const c_char;
    pub fn trn_device_cu_count(count: *mut c_int) -> trn_status;
    pub fn trn_set_tuning(key: *const c_char, value: c_int) -> trn_status;
}
