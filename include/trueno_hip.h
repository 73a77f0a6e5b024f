/* trueno_hip.h - C ABI of libtrueno_hip.so: the MI355X (gfx950) backend for trueno-gpu's fused
 * k-quant matrix path.
 *
 * What binds here.  trueno-gpu reaches its GPU through a table of 25 `cu*` function pointers
 * (trueno-gpu/src/driver/sys.rs:99-201) loaded from libcuda (sys.rs:230-257).  Sections 1-6 below
 * are a one-to-one image of that table over the HIP runtime, so `driver/sys.rs` can bind this
 * library instead and `driver/{context,module,stream,memory}.rs` stay as they are.  Section 7
 * replaces "emit PTX, JIT it" (kernels/mod.rs:56-67 + driver/module.rs:62-79) by a code object that
 * ships inside the library.  Section 8 are typed launchers for the kernels of
 * trueno-gpu/src/kernels/quantize.rs; they own the launch geometry.  Sections 9-10 have no
 * counterpart in the reference (timing and a test surface).
 *
 * Conventions.  Every call returns a status: 0 = success, otherwise the hipError_t value (the
 * reference maps any non-zero CUresult to GpuError::CudaDriver(name, code), sys.rs:360-369; a missing
 * device is hipErrorNoDevice = 100, which maps to GpuError::CudaNotAvailable).  Device pointers
 * are plain 64-bit integers (CUdeviceptr, sys.rs:60).  The library never owns host memory and never
 * keeps a host pointer after a synchronous call returns.  Device memory for the caller's data comes
 * from trn_mem_alloc only.  Beside it the library keeps scratch of its own, per (device, stream),
 * allocated on first use and freed with the stream: the partial sums and arrival counters of the
 * products that are cut along K (trn_q*k_gemm, trn_gemv_f32, trn_incremental_attention), the tables
 * of a list's launches of more than sixteen entries (trn_kquant_gemv_batch), the tables of the
 * resident executor (batch_mode 1); and one static array of 16 MiB + 64 KiB per GPU
 * (trn_q4k_gemm_noalloc).  The calls that never allocate: the GEMV launchers, trn_kquant_gemv_batch
 * for lists whose launches hold at most sixteen entries or while the stream is being captured,
 * trn_q4k_gemm_noalloc, the element-wise launchers.  All entry points may be called from any thread;
 * calls that touch a device act on the calling thread's current device (trn_ctx_set_current).
 */
#ifndef TRUENO_HIP_H
#define TRUENO_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TRN_API __attribute__((visibility("default")))

typedef int trn_status;                 /* CUresult,    sys.rs:27  */
typedef int trn_device;                 /* CUdevice,    sys.rs:33  */
typedef struct trn_ctx_s* trn_ctx;      /* CUcontext,   sys.rs:39  */
typedef struct trn_module_s* trn_module;     /* CUmodule,    sys.rs:45 */
typedef struct trn_function_s* trn_function; /* CUfunction,  sys.rs:51 */
typedef void* trn_stream;               /* CUstream,    sys.rs:57 (NULL = default stream) */
typedef uint64_t trn_dptr;              /* CUdeviceptr, sys.rs:60 */
typedef struct trn_event_s* trn_event;

#define TRN_SUCCESS 0
#define TRN_ERROR_INVALID_VALUE 1       /* hipErrorInvalidValue */
#define TRN_ERROR_NO_DEVICE 100         /* hipErrorNoDevice */
#define TRN_ERROR_INVALID_DEVICE 101    /* hipErrorInvalidDevice */
#define TRN_ERROR_NOT_FOUND 500         /* hipErrorNotFound */
/* Not a hipError_t: a device-side wait of the resident list executor (batch_mode 1) ran out of its spin budget and
 * the kernel gave up.  Reported once, by the next trn_stream_synchronize / trn_event_synchronize /
 * trn_ctx_synchronize / trn_stream_destroy / trn_kquant_gemv_batch on that stream; the outputs of that list are
 * not valid.  The context stays usable. */
#define TRN_ERROR_WAIT_ABANDONED 9001
/* Not a hipError_t: trn_q4k_gemm_noalloc was asked for a product whose partial results do not fit the library's
 * static scratch buffer.  Nothing was launched. */
#define TRN_ERROR_SCRATCH_TOO_SMALL 9002
#define TRN_STREAM_NON_BLOCKING 1u      /* CU_STREAM_NON_BLOCKING, driver/stream.rs:60 */

/* ---- 1. initialisation (sys.rs:101-102) ------------------------------------------------ */
TRN_API trn_status trn_init(unsigned flags);                                    /* cuInit */

/* ---- 2. devices (sys.rs:104-114) --------------------------------------------------------- */
TRN_API trn_status trn_device_get_count(int* count);                            /* cuDeviceGetCount */
TRN_API trn_status trn_device_get(trn_device* device, int ordinal);             /* cuDeviceGet */
TRN_API trn_status trn_device_get_name(char* name, int len, trn_device device); /* cuDeviceGetName */
TRN_API trn_status trn_device_total_mem(size_t* bytes, trn_device device);      /* cuDeviceTotalMem_v2 */

/* ---- 3. primary context (sys.rs:116-126) -------------------------------------------------- */
TRN_API trn_status trn_primary_ctx_retain(trn_ctx* ctx, trn_device device);     /* cuDevicePrimaryCtxRetain */
TRN_API trn_status trn_primary_ctx_release(trn_device device);                  /* cuDevicePrimaryCtxRelease */
TRN_API trn_status trn_ctx_set_current(trn_ctx ctx);                            /* cuCtxSetCurrent */
TRN_API trn_status trn_ctx_synchronize(void);                                   /* cuCtxSynchronize */

/* ---- 4. modules (sys.rs:128-140) ----------------------------------------------------------- */
/* image: a gfx950 code object (ELF) in host memory, where the reference passes PTX text. */
TRN_API trn_status trn_module_load_data(trn_module* module, const void* image); /* cuModuleLoadData */
TRN_API trn_status trn_module_unload(trn_module module);                        /* cuModuleUnload */
TRN_API trn_status trn_module_get_function(trn_function* func, trn_module module,
                                           const char* name);                   /* cuModuleGetFunction */
/* The reference compiles some kernel parameters into the PTX of one kernel instance: RmsNormKernel::new(hidden_size)
 * .with_epsilon(e) (layernorm.rs:388-431), FusedResidualRmsNormKernel (elementwise.rs:109-149) and
 * IncrementalAttentionKernel::new / ::with_gqa (attention.rs:808-901).  A pre-built code object cannot, so they are
 * set on the function handle (one module per kernel instance, as in the reference) before it is launched by name with
 * the reference's own parameter list: "rmsnorm" (input, output, gamma), "fused_residual_rmsnorm" (residual, input,
 * output, gamma), "incremental_attention" (q, k, v, out, seq_len).  Launching one of these by name without its
 * constants returns TRN_ERROR_INVALID_VALUE; nothing beyond the reference's parameters is ever read.  The constants
 * belong to the one handle that trn_module_get_function returns for (module, name): two kernel instances with
 * different constants need a module each, and a thread that sets a handle while another launches it must be kept
 * apart from it by the caller (a set is two or five plain stores). */
TRN_API trn_status trn_function_set_rmsnorm(trn_function func, uint32_t hidden_size, float epsilon);
TRN_API trn_status trn_function_set_attention(trn_function func, uint32_t head_dim, uint32_t num_heads,
                                              uint32_t num_kv_heads, uint32_t max_seq_len, float scale);

/* ---- 5. memory (sys.rs:142-176) ------------------------------------------------------------ */
TRN_API trn_status trn_mem_alloc(trn_dptr* ptr, size_t size);                   /* cuMemAlloc_v2 */
TRN_API trn_status trn_mem_free(trn_dptr ptr);                                  /* cuMemFree_v2; 0 is a no-op */
TRN_API trn_status trn_memcpy_htod(trn_dptr dst, const void* src, size_t size); /* cuMemcpyHtoD_v2 */
TRN_API trn_status trn_memcpy_dtoh(void* dst, trn_dptr src, size_t size);       /* cuMemcpyDtoH_v2 */
TRN_API trn_status trn_memcpy_htod_async(trn_dptr dst, const void* src, size_t size, trn_stream stream); /* cuMemcpyHtoDAsync_v2 */
TRN_API trn_status trn_memcpy_dtoh_async(void* dst, trn_dptr src, size_t size, trn_stream stream);       /* cuMemcpyDtoHAsync_v2 */
TRN_API trn_status trn_memcpy_dtod(trn_dptr dst, trn_dptr src, size_t size);    /* cuMemcpyDtoD_v2 */
TRN_API trn_status trn_memcpy_dtod_async(trn_dptr dst, trn_dptr src, size_t size, trn_stream stream);    /* cuMemcpyDtoDAsync_v2 */
TRN_API trn_status trn_mem_get_info(size_t* free_bytes, size_t* total_bytes);   /* cuMemGetInfo_v2 */

/* ---- 6. streams and launch (sys.rs:178-200) -------------------------------------------------- */
TRN_API trn_status trn_stream_create(trn_stream* stream, unsigned flags);       /* cuStreamCreate */
TRN_API trn_status trn_stream_destroy(trn_stream stream);                       /* cuStreamDestroy_v2 */
TRN_API trn_status trn_stream_synchronize(trn_stream stream);                   /* cuStreamSynchronize */
/* cuLaunchKernel.  kernel_params[i] points at a host copy of parameter i, in declared order
 * (driver/stream.rs:110-154).  For the k-quant kernels of the built-in module the grid, block and
 * shared-memory arguments are ignored and replaced by the kernel's own geometry (the reference's
 * documented grid = N blocks of 32 threads, quantize.rs:1151-1155, is a warp32 shape); the result
 * never depends on the geometry the caller passed.  The same holds for a module made by trn_module_load_data from
 * the image trn_builtin_image returns.  Kernels of the built-in code object that are not reference names are
 * internal: launching one by name returns TRN_ERROR_INVALID_VALUE.  Functions of any other module launch exactly
 * as given. */
TRN_API trn_status trn_launch_kernel(trn_function func, unsigned grid_x, unsigned grid_y, unsigned grid_z,
                                     unsigned block_x, unsigned block_y, unsigned block_z,
                                     unsigned shared_mem_bytes, trn_stream stream,
                                     void** kernel_params, void** extra);

/* ---- 7. the built-in code object ------------------------------------------------------------- */
/* Loads the gfx950 code object embedded in this library on the current device.  Stands where the
 * reference does CudaModule::from_ptx(&ctx, &kernel.emit_ptx()) (driver/module.rs:62-79,
 * kernels/mod.rs:65-67).  It exports, with the reference's parameter lists:
 *   q4k_gemv_warp_reduce  q5k_gemv_warp_reduce  q6k_gemv_warp_reduce   (y, w, x, k_dim, n_dim)
 *   q4k_gemm_ggml         q5k_gemm_ggml         q6k_gemm_ggml          (a, b_quant, c, m, n, k)
 *   q4k_gemm_fused                                                      (a, b_quant, c, m, n, k) */
TRN_API trn_status trn_module_load_builtin(trn_module* module);
/* Pointer to and size of that embedded code object (for callers that want trn_module_load_data; the module is
 * recognised and treated like trn_module_load_builtin's). */
TRN_API trn_status trn_builtin_image(const void** image, size_t* size);

/* ---- 8. typed launchers ------------------------------------------------------------------------
 * y[n] = sum_k dequant(W)[n,k] * x[k].  W: n rows x (k/256) super-blocks, row-major, 144/176/210
 * bytes per super-block; x: k f32; y: n f32.  k must be a multiple of 256 (else
 * TRN_ERROR_INVALID_VALUE); n = 0 is a no-op; k = 0 writes zeros.  Asynchronous on `stream`.
 * Replace Q4KGemvKernel / Q5KGemvKernel / Q6KGemvKernel + launch_kernel
 * (quantize.rs:1156-1523, :1532-1724, :1733-1965). */
TRN_API trn_status trn_q4k_gemv(trn_stream stream, trn_dptr y, trn_dptr w, trn_dptr x, uint32_t k, uint32_t n);
TRN_API trn_status trn_q5k_gemv(trn_stream stream, trn_dptr y, trn_dptr w, trn_dptr x, uint32_t k, uint32_t n);
TRN_API trn_status trn_q6k_gemv(trn_stream stream, trn_dptr y, trn_dptr w, trn_dptr x, uint32_t k, uint32_t n);
/* C[m x n] = A[m x k] . dequant(W[n x k])^T, c[row*n + col]; A, C f32 row-major.  The decode is the
 * GEMV-family one, so m = 1 equals the GEMV.  Replace QuantizeKernel::ggml / Q5KKernel / Q6KKernel
 * (quantize.rs:347-579, :640-866, :926-1121).  Which kernel takes a product is the library's choice by its shape (one
 * token: the GEMV engine; Q4_K, two to four tokens, k <= 4096: the integer matrix cores where that is fastest; otherwise
 * the f16 matrix cores, or for a few tokens against a small matrix the GEMV engine once per token); every one of them is
 * within the 1e-5 relative L2 of fp64 and no worse than an f32 evaluation in the reference's order, but they are not
 * bit-identical to each other.  An infinity or NaN among a token's activations makes that token's results non-finite
 * (NaN where the reference's sum would give an infinity) and leaves the other tokens alone. */
TRN_API trn_status trn_q4k_gemm(trn_stream stream, trn_dptr a, trn_dptr b_quant, trn_dptr c, uint32_t m, uint32_t n, uint32_t k);
TRN_API trn_status trn_q5k_gemm(trn_stream stream, trn_dptr a, trn_dptr b_quant, trn_dptr c, uint32_t m, uint32_t n, uint32_t k);
TRN_API trn_status trn_q6k_gemm(trn_stream stream, trn_dptr a, trn_dptr b_quant, trn_dptr c, uint32_t m, uint32_t n, uint32_t k);

/* trn_q4k_gemm for callers that cannot allocate device memory: code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc.  No counterpart in the reference.  Same arguments, same kernels and bit-identical
 * results; but where trn_q4k_gemm keeps a per-stream scratch buffer that it allocates and grows on demand (partial
 * results of the parts of K and their arrival counters), this entry point uses a buffer that is part of the library
 * image: a static device array of 16 MiB + 64 KiB, of which every GPU the library runs on holds one copy until the
 * process ends.  After the library's first use on the device (any launcher, or trn_ctx_set_current, loads the kernels
 * and looks the buffer's address up once) it calls nothing that allocates or frees.  The product is cut exactly as
 * trn_q4k_gemm would cut it - hence the same bits - and when that cut needs more scratch than the buffer holds the call
 * returns TRN_ERROR_SCRATCH_TOO_SMALL and launches nothing; no other failure is reported under that name (every cut that
 * the library chooses by itself needs at most 11.2 MB on 256 CUs; a cut forced with trn_set_tuning may need more; m = 1
 * and unaligned operands take kernels that need no scratch).  All calls on
 * one GPU share that GPU's buffer: calls that overlap in time on different streams of one GPU race - keep them on
 * one stream, or order the streams.  The kernels leave the counters at zero for the next call. */
TRN_API trn_status trn_q4k_gemm_noalloc(trn_stream stream, trn_dptr a, trn_dptr b_quant, trn_dptr c, uint32_t m, uint32_t n, uint32_t k);

/* The same products with the GEMM family's weight decode AS WRITTEN in the reference (quantize.rs:445-514 Q4_K,
 * :727-807 Q5_K, :1009-1064 Q6_K: contiguous 12-bit scale fields normalised by 1/63, sequential nibbles, Q6_K's unsigned
 * scales and q = ql + 4*q2 - 32), i.e. policy 1 of the dequantise surface below; the contraction is the intended one
 * (a dot product per (row, col), quantize.rs:568-574).  trn_q*k_gemm above use the canonical (GGML) decode, so that
 * m = 1 equals the GEMV; these exist so that q4k_gemm_ggml / q5k_gemm_ggml / q6k_gemm_ggml can be run against their
 * as-written decode too.  Value-by-value kernels (one wave per row of W): correct, not fast. */
TRN_API trn_status trn_q4k_gemm_as_written(trn_stream stream, trn_dptr a, trn_dptr b_quant, trn_dptr c, uint32_t m, uint32_t n, uint32_t k);
TRN_API trn_status trn_q5k_gemm_as_written(trn_stream stream, trn_dptr a, trn_dptr b_quant, trn_dptr c, uint32_t m, uint32_t n, uint32_t k);
TRN_API trn_status trn_q6k_gemm_as_written(trn_stream stream, trn_dptr a, trn_dptr b_quant, trn_dptr c, uint32_t m, uint32_t n, uint32_t k);

/* The legacy 18-byte-block "simplified" Q4_K GEMM, kernel name q4k_gemm_fused: W is n rows x (k/32) blocks
 * (f16 scale + 16 bytes of nibbles, w = scale * q), k a multiple of 32, C as above.  Replaces
 * QuantizeKernel::new (quantize.rs:84-93, :151-336). */
TRN_API trn_status trn_q4k_gemm_fused(trn_stream stream, trn_dptr a, trn_dptr b_quant, trn_dptr c, uint32_t m, uint32_t n, uint32_t k);

/* A list of GEMVs issued with one call, in order, on one stream: the weight pass of a decode step
 * (the caller in the reference issues one launch_kernel per matrix per token, docs/roadmaps/
 * roadmap.yaml:359-368).  Entry i computes y = dequant(W) x exactly as the typed launcher of its
 * format would; a later entry may read what an earlier one wrote (the library finds those
 * dependencies from the pointer ranges).  fmt: 4 = Q4_K, 5 = Q5_K, 6 = Q6_K.
 * By default (mode 0) entries that do not touch one another's vectors share a launch: the first entry still
 * waiting, plus every later one of the list (q, k, v of a decoder layer; gate and up; the same of other layers
 * when each layer has activation buffers of its own; ...) that depends neither on it nor on anything it would
 * overtake.  Up to sixteen entries travel in the kernel's arguments; a launch of more takes them from tables in
 * device memory, which are made when a list is first seen on a stream and kept for as long as the same list (the
 * same descriptors, byte for byte) comes again - up to eight lists per stream, the one used longest ago makes room.
 * While the stream is being captured into a graph nothing is copied or allocated: a list that the same stream has
 * issued eagerly before (and whose tables it still holds) is recorded with those launches, and the tables a graph
 * reads are then kept until the process ends (a few hundred KB per captured list); any other list is recorded as
 * launches of at most sixteen entries.  What an entry computes does not depend on the company it is launched in: the results are, bit for
 * bit, those of one launch per entry in list order.
 * With trn_set_tuning("batch_mode", 1), and when every entry meets the fast kernels' alignment (x 16 B,
 * W 16 B / 2 B for Q6_K), the list runs as ONE cooperative launch of resident workgroups: the list is cut in
 * phases of mutually independent entries with a device-side barrier between phases.  This form keeps, per
 * (device, stream), small device buffers with the list, the work assignment and the barrier counters (allocated on
 * first use, kept until the stream is destroyed); a list identical to the previous one on that stream is not uploaded
 * again.  If a device-side wait ever runs out of its (seconds-long) spin budget the kernel exits and the next
 * synchronising call on that stream returns TRN_ERROR_WAIT_ABANDONED.  Both forms give bit-identical results. */
/* An entry may fold the element-wise steps of a decoder layer in (zero pointers: absent):
 *   x'  = x                          or silu(x) * x2            (TRN_GEMV_SWIGLU_INPUT; x = gate, x2 = up: fused_swiglu)
 *   x'' = x' * gamma                 (gamma: k f32, the weights of rmsnorm)
 *   y   = s * (W . x'') + residual   (residual: n f32; may be y itself),
 *         s = 1, or 1 / sqrt(mean(x'^2) + norm_eps) with TRN_GEMV_NORM_INPUT (norm_eps 0 = 1e-6)
 * so that rmsnorm -> projection, fused_residual_rmsnorm's second half, swiglu -> down projection and the residual
 * add after o / down need no launches of their own.  gamma, x2 and residual count as read by the dependency
 * analysis.  Such entries need x, x2 and gamma 16-byte aligned. */
#define TRN_GEMV_NORM_INPUT 1u   /* the entry reads x' / sqrt(mean(x'^2) + eps) instead of x' */
#define TRN_GEMV_SWIGLU_INPUT 8u /* the entry reads silu(x) * x2 instead of x */
typedef struct trn_gemv_desc {
  uint32_t fmt;
  uint32_t k;
  uint32_t n;
  uint32_t flags;      /* 0 or TRN_GEMV_NORM_INPUT | TRN_GEMV_SWIGLU_INPUT */
  trn_dptr y;
  trn_dptr w;
  trn_dptr x;
  trn_dptr gamma;
  trn_dptr x2;
  trn_dptr residual;
  float norm_eps;
  uint32_t reserved;   /* 0 */
} trn_gemv_desc;
TRN_API trn_status trn_kquant_gemv_batch(trn_stream stream, const trn_gemv_desc* descs, uint32_t count);
/* Which launch of mode 0 each entry of the list would go into: launch_of[i] = 0, 1, ... in launch order.  Launches
 * nothing (for tools that want to time or describe the launches of a list; no counterpart in the reference). */
TRN_API trn_status trn_kquant_gemv_plan(const trn_gemv_desc* descs, uint32_t count, uint32_t* launch_of);

/* ---- 9. test surface: dequantise to f32 (no counterpart in the reference) ------------------------
 * out[sb*256 + i] = weight i of super-block sb.  policy 0 = GEMV-family decode
 * (quantize.rs:1237-1483, :1589-1693, :1806-1934); policy 1 = GEMM-family decode as written
 * (quantize.rs:445-514, :727-807, :1009-1064). */
TRN_API trn_status trn_q4k_dequant_f32(trn_stream stream, trn_dptr out, trn_dptr w, uint64_t n_sb, int policy);
TRN_API trn_status trn_q5k_dequant_f32(trn_stream stream, trn_dptr out, trn_dptr w, uint64_t n_sb, int policy);
TRN_API trn_status trn_q6k_dequant_f32(trn_stream stream, trn_dptr out, trn_dptr w, uint64_t n_sb, int policy);
/* out[b*32 + i] = weight i of simplified block b (quantize.rs:237-267). */
TRN_API trn_status trn_q4k_simplified_dequant_f32(trn_stream stream, trn_dptr out, trn_dptr w, uint64_t n_blocks);

/* ---- 10. timing, errors, tuning (no counterpart in the reference) --------------------------------- */
TRN_API trn_status trn_event_create(trn_event* event);
TRN_API trn_status trn_event_destroy(trn_event event);
TRN_API trn_status trn_event_record(trn_event event, trn_stream stream);
TRN_API trn_status trn_event_synchronize(trn_event event);
TRN_API trn_status trn_event_elapsed_ms(float* ms, trn_event start, trn_event stop);
/* Single-query attention over a KV cache, the step between the q/k/v and the o projection of a decoding layer:
 *   out[h] = sum_i softmax_i(scale * q[h] . k[kv(h)][i]) v[kv(h)][i],  i < seq_len,  kv(h) = h * num_kv_heads / num_heads
 *   q, out: [num_heads][head_dim] f32;  k, v: [num_kv_heads][max_seq_len][head_dim] f32.
 * trueno-gpu/src/kernels/attention.rs:808-1095 (IncrementalAttentionKernel, "incremental_attention", parameters
 * (q_ptr, k_ptr, v_ptr, out_ptr, seq_len); head_dim, the head counts, max_seq_len and scale are compiled into its
 * PTX: here they are arguments of the typed launcher, and constants of the function handle for a by-name launch,
 * trn_function_set_attention).  The reference's kernel covers head_dim <= 64;
 * this one head_dim % 4 == 0 up to 256.  1 <= seq_len <= max_seq_len; pointers 16-byte aligned.  Keeps a small
 * per-stream workspace (allocated on first use). */
TRN_API trn_status trn_incremental_attention(trn_stream stream, trn_dptr q, trn_dptr k, trn_dptr v, trn_dptr out,
                                             uint32_t seq_len, uint32_t head_dim, uint32_t num_heads, uint32_t num_kv_heads,
                                             uint32_t max_seq_len, float scale);

/* Re-packs n_sb GGML Q5_K blocks (what a GGUF file holds: d, dmin, scales[12], qh[32], qs[128]) into the Q5_K
 * layout of the reference's kernels (trueno-gpu/src/kernels/quantize.rs:1589-1693, which is not GGML's); the
 * dequantised values are unchanged.  dst may be src.  Q4_K and Q6_K need no such step: the reference reads GGML's
 * bytes as they are.  No counterpart in the reference: its callers re-pack on the host. */
TRN_API trn_status trn_q5k_from_ggml(trn_stream stream, trn_dptr dst, trn_dptr src, uint64_t n_sb);

/* f32 GEMV: y[n] = sum_k a[k*n_dim + n] * x[k]; a is K x N row-major, i.e. transposed relative to the quantized
 * matrices.  trueno-gpu/src/kernels/gemv.rs: GemvKernel "gemv_warp_reduce" :21-166 and CoalescedGemvKernel
 * "gemv_coalesced" :188-398, both (y_ptr, a_ptr, x_ptr, k_dim, n_dim); the built-in module has both names.  Keeps a
 * small per-stream workspace (allocated on first use). */
TRN_API trn_status trn_gemv_f32(trn_stream stream, trn_dptr y, trn_dptr a, trn_dptr x, uint32_t k, uint32_t n);

/* ---- element-wise steps between the GEMVs of a decoder layer (f32 vectors) ---------------------------------
 * The same kernels are in the built-in module under the reference's names "residual_add", "fused_swiglu",
 * "rmsnorm", "fused_residual_rmsnorm", all with the reference's parameter lists.  The reference compiles hidden_size
 * and epsilon of the two norms into its PTX; for a by-name launch they are constants of the function handle
 * (trn_function_set_rmsnorm).  Whatever grid and block a by-name launch passes is replaced. */
/* output[i] = input1[i] + input2[i]; output may alias an input.  trueno-gpu/src/kernels/elementwise.rs:33-101 */
TRN_API trn_status trn_residual_add(trn_stream stream, trn_dptr input1, trn_dptr input2, trn_dptr output, uint32_t n);
/* output[i] = silu(gate[i]) * up[i], silu(g) = g / (1 + 2^(-g * 1.442695f)).  elementwise.rs:521-592 */
TRN_API trn_status trn_fused_swiglu(trn_stream stream, trn_dptr gate, trn_dptr up, trn_dptr output, uint32_t n);
/* One row: output[i] = input[i] * rsqrt(mean(input^2) + epsilon) * gamma[i]; output may alias input.
 * trueno-gpu/src/kernels/layernorm.rs:388-516 (RmsNormKernel; its default epsilon is 1e-5, :400-405) */
TRN_API trn_status trn_rmsnorm(trn_stream stream, trn_dptr input, trn_dptr output, trn_dptr gamma, uint32_t hidden_size,
                               float epsilon);
/* One row: the same with x = residual + input; output may alias residual.  elementwise.rs:109-248 */
TRN_API trn_status trn_fused_residual_rmsnorm(trn_stream stream, trn_dptr residual, trn_dptr input, trn_dptr output,
                                              trn_dptr gamma, uint32_t hidden_size, float epsilon);

/* dst[0..bytes) = src[0..bytes) with one 16-byte load and store per lane; bytes % 16 == 0.
 * The plain-copy yardstick that HBM counters are scaled by. */
TRN_API trn_status trn_copy_u128(trn_stream stream, trn_dptr dst, trn_dptr src, uint64_t bytes);
/* Reads src[0..bytes) once with non-temporal 16-byte loads, eight in flight per lane, and stores nothing (one word of `sink`, 4 bytes,
 * is written only if the XOR of everything read equals one particular value); bytes % 16 == 0.  The read-only
 * yardstick: what one launch over that many bytes costs when nothing is computed.  No counterpart in the reference. */
TRN_API trn_status trn_read_u128(trn_stream stream, trn_dptr src, uint64_t bytes, trn_dptr sink);
TRN_API const char* trn_error_name(trn_status status);
TRN_API const char* trn_error_string(trn_status status);
/* Number of compute units of the current device (sizes the launches). */
TRN_API trn_status trn_device_cu_count(int* count);
/* Launch tuning knobs, process-wide (for tests and measurements; atomics, no other synchronisation); 0 restores the default.  "gemv_blocks_per_cu", "gemv_row_groups":
 * geometry of the single-GEMV kernels.  "batch_mode": how trn_kquant_gemv_batch runs a list - 0 grouped
 * launches (default), 1 one cooperative launch of resident workgroups with device-side barriers.
 * "chain_spin_limit": polls a device-side barrier wait may take before it gives up.
 * "group_off": 1 = in mode 0 one launch per entry; "group_max": most entries in a launch (0 = as many as the list offers,
 * up to 4096; 16 or less keeps every launch on the kernel-argument form); "group_window": how far down the list a launch
 * looks for entries (0 = twice group_max); "group_waves": least waves per workgroup of a launch of up to sixteen entries (0 = 8,
 * or what its widest entry needs); "many_waves": waves per workgroup of a launch of more than sixteen entries (0 = 12);
 * "group_slab_weight": percent added to an entry's bytes per further 4096 columns when a launch of up to sixteen entries
 * shares out its workgroups (0 = 40); "many_slab_weight": the same for a launch of more than sixteen (0 = 13);
 * "many_item_kb": what every piece of an entry costs the workgroup that takes it, in KB of weights (0 = 64).
 * "gemv_stream_off": 1 = no matrix streams its rows through LDS (every GEMV loads its rows into registers straight from
 * memory; same bits); "gemv_stream_q6k": 1 = Q6_K matrices of up to 4096 columns stream too (their slots are larger:
 * in a launch of more than sixteen entries only with "many_waves" of 10 or less; 4-7 % faster on long lists at 8);
 * "gemv_stream_waves": waves per workgroup of a single streamed GEMV (0 = 4); "gemv_stream_min_rows": a single GEMV
 * streams when a wave gets at least this many rows (0 = 16); "group_stream_min_rows": the same for an entry of a launch
 * of up to sixteen entries (0 = 24); "gemv_stream_cost": percent of its bytes a streamed entry
 * counts for when a launch shares out its workgroups (0 = 95).
 * "gemm_few": the Q4_K product of two to four tokens on the integer matrix cores - 0 = where its estimated time is the
 * lowest, 1 = wherever it can run, 2 = never.
 * "gemm_mfma_off": 1 = the k-quant GEMMs never take the f16 matrix-core form; "gemm_k_parts": into how many parts
 * that form cuts K; "gemm_waves": 4, 8 or (Q4_K) 12 strips of 32 rows per workgroup; "gemm_tiles": 1 or 2 tiles of 16 tokens per
 * workgroup (0 for each of the three = chosen from the shape by an estimated time; any of them set also keeps a
 * product of a few tokens on the matrix cores);
 * "attention_per_cu": workgroups per CU the single-query attention aims at (0 = 2); "attention_min_steps": least
 * number of steps (of 8 positions at head_dim 128) in a chunk of positions (0 = 8). */
TRN_API trn_status trn_set_tuning(const char* key, int value);

#ifdef __cplusplus
}
#endif
#endif /* TRUENO_HIP_H */
