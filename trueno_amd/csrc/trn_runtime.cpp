// libtrueno_hip.so: the C ABI of include/trueno_hip.h over the HIP runtime.
//
// Host-only C++ (no device code in this file).  The gfx950 kernels live in a code object that
// the build embeds below; every launch, typed or by name, goes through hipModuleLaunchKernel on
// functions of that code object.  There is no CPU fallback anywhere: without a device every
// entry point that needs one returns the HIP error (hipErrorNoDevice = 100).
//
// Mirrors trueno-gpu/src/driver/sys.rs:99-201 (the cu* table) entry by entry.
#include "../../include/trueno_hip.h"

#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <string>

// ---- embedded code object -------------------------------------------------------------------
#ifndef TRN_HSACO_PATH
#error "TRN_HSACO_PATH must name the gfx950 code object to embed"
#endif
asm(".section .rodata\n"
    ".balign 4096\n"
    ".global trn_builtin_hsaco_begin\n"
    "trn_builtin_hsaco_begin:\n"
    ".incbin \"" TRN_HSACO_PATH "\"\n"
    ".global trn_builtin_hsaco_end\n"
    "trn_builtin_hsaco_end:\n"
    ".byte 0\n"
    ".previous\n");
extern "C" const unsigned char trn_builtin_hsaco_begin[];
extern "C" const unsigned char trn_builtin_hsaco_end[];

namespace {

enum Fmt { Q4K = 0, Q5K = 1, Q6K = 2, NFMT = 3 };
const char* const kFmtName[NFMT] = {"q4k", "q5k", "q6k"};
const uint32_t kSbBytes[NFMT] = {144, 176, 210};

// kinds of functions the launch-by-name path recognises
enum Kind { KIND_OTHER = 0, KIND_GEMV = 1, KIND_GEMM = 2 };

constexpr int kMaxDevices = 64;
constexpr uint32_t kGemvRowsPerBatch = 2;     // U of the fast GEMV kernel
constexpr uint32_t kFastLdsLimit = 64 * 1024;  // dynamic LDS the fast kernels may ask for

struct DeviceKernels {
  bool loaded = false;
  hipModule_t module = nullptr;
  int cu_count = 0;
  hipFunction_t gemv_fast[NFMT] = {}, gemv_generic[NFMT] = {};
  hipFunction_t gemm_fast[NFMT] = {}, gemm_generic[NFMT] = {};
  hipFunction_t dequant_fast[NFMT] = {}, dequant_generic[NFMT] = {};
  hipFunction_t copy_u128 = nullptr;
};

std::mutex g_mutex;
DeviceKernels g_dev[kMaxDevices];
int g_tune_blocks_per_cu = 0;
int g_tune_row_groups = 0;

inline trn_status st(hipError_t e) { return static_cast<trn_status>(e); }

#define TRN_TRY(expr)                         \
  do {                                        \
    hipError_t trn_e_ = (expr);               \
    if (trn_e_ != hipSuccess) return st(trn_e_); \
  } while (0)

hipError_t get_fn(hipModule_t m, hipFunction_t* f, const std::string& name) {
  return hipModuleGetFunction(f, m, name.c_str());
}

// Kernels of the built-in code object on the calling thread's current device, loaded on first use.
hipError_t device_kernels(DeviceKernels** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
  std::lock_guard<std::mutex> lock(g_mutex);
  DeviceKernels& d = g_dev[dev];
  if (!d.loaded) {
    hipModule_t m = nullptr;
    if ((e = hipModuleLoadData(&m, trn_builtin_hsaco_begin)) != hipSuccess) return e;
    DeviceKernels t;
    t.module = m;
    for (int f = 0; f < NFMT; ++f) {
      const std::string p = kFmtName[f];
      if ((e = get_fn(m, &t.gemv_fast[f], p + "_gemv_warp_reduce")) != hipSuccess ||
          (e = get_fn(m, &t.gemv_generic[f], p + "_gemv_generic")) != hipSuccess ||
          (e = get_fn(m, &t.gemm_fast[f], p + "_gemm_ggml")) != hipSuccess ||
          (e = get_fn(m, &t.gemm_generic[f], p + "_gemm_generic")) != hipSuccess ||
          (e = get_fn(m, &t.dequant_fast[f], p + "_dequant_f32")) != hipSuccess ||
          (e = get_fn(m, &t.dequant_generic[f], p + "_dequant_f32_generic")) != hipSuccess) {
        (void)hipModuleUnload(m);
        return e;
      }
    }
    if ((e = get_fn(m, &t.copy_u128, "kq_copy_u128")) != hipSuccess) {
      (void)hipModuleUnload(m);
      return e;
    }
    if ((e = hipDeviceGetAttribute(&t.cu_count, hipDeviceAttributeMultiprocessorCount, dev)) != hipSuccess) {
      (void)hipModuleUnload(m);
      return e;
    }
    if (t.cu_count <= 0) t.cu_count = 256;
    t.loaded = true;
    d = t;
  }
  *out = &d;
  return hipSuccess;
}

// Geometry of the fast GEMV kernel for an n x k matrix.  The kernel accepts any grid and any
// block that is a multiple of 64; this picks a good one and the LDS it needs.
struct GemvGeometry {
  uint32_t grid = 0, block = 0, lds = 0;
  bool fits = false;
};

GemvGeometry gemv_geometry(const DeviceKernels& d, uint32_t k, uint32_t n) {
  GemvGeometry g;
  const uint32_t nsb = k / 256u;
  const uint32_t slabs = (nsb + 15u) / 16u;
  const uint32_t sw = std::min<uint32_t>(slabs, 8u);
  uint32_t groups = g_tune_row_groups > 0 ? uint32_t(g_tune_row_groups) : std::max<uint32_t>(1u, 4u / sw);
  groups = std::max<uint32_t>(1u, std::min<uint32_t>(groups, 8u / sw));
  const uint32_t ug = kGemvRowsPerBatch * groups;
  const uint32_t per_cu = g_tune_blocks_per_cu > 0 ? uint32_t(g_tune_blocks_per_cu) : 4u;
  const uint64_t target_blocks = uint64_t(d.cu_count) * per_cu;
  uint64_t rows = (uint64_t(n) + target_blocks - 1) / target_blocks;
  rows = std::max<uint64_t>(ug, (rows + ug - 1) / ug * ug);
  // keep activations + partial sums within the LDS the kernel may ask for
  const uint64_t x_bytes = uint64_t(k) * 4u;
  if (x_bytes + uint64_t(sw) * ug * 4u > kFastLdsLimit) return g;
  const uint64_t max_rows = (kFastLdsLimit - x_bytes) / (uint64_t(sw) * 4u) / ug * ug;
  rows = std::min<uint64_t>(rows, max_rows);
  g.grid = uint32_t((uint64_t(n) + rows - 1) / rows);
  // the kernel recomputes rows-per-block from the grid; it can only come out <= rows
  g.block = 64u * sw * groups;
  g.lds = uint32_t(x_bytes + uint64_t(sw) * rows * 4u);
  g.fits = true;
  return g;
}

bool aligned(uint64_t p, uint64_t a) { return (p & (a - 1)) == 0; }

bool gemv_fast_ok(Fmt f, uint64_t y, uint64_t w, uint64_t x) {
  // 128-bit activation loads; Q4_K/Q5_K blocks are streamed with aligned 128-bit loads (their
  // rows are multiples of 16 bytes); Q6_K blocks (210 bytes) only need their natural 2 bytes.
  return aligned(x, 16) && aligned(y, 4) && aligned(w, f == Q6K ? 2 : 16);
}

hipError_t launch_gemm_like(Fmt f, hipStream_t stream, uint64_t a, uint64_t w, uint64_t c, uint32_t m, uint32_t n,
                            uint32_t k, bool is_gemv) {
  if (k % 256u != 0) return hipErrorInvalidValue;
  if (n == 0 || m == 0) return hipSuccess;
  if ((a == 0 && k != 0) || c == 0 || (w == 0 && k != 0)) return hipErrorInvalidValue;
  DeviceKernels* d = nullptr;
  hipError_t e = device_kernels(&d);
  if (e != hipSuccess) return e;
  const uint32_t grid_y = std::min<uint32_t>(m, 65535u);
  // GEMV parameter order is (y, w, x, k, n); GEMM is (a, b_quant, c, m, n, k)
  void* gemv_args[] = {&c, &w, &a, &k, &n};
  void* gemm_args[] = {&a, &w, &c, &m, &n, &k};
  void** args = is_gemv ? gemv_args : gemm_args;
  GemvGeometry g;
  if (k != 0 && gemv_fast_ok(f, c, w, a) && (is_gemv || (aligned(uint64_t(k) * 4u, 16) && aligned(uint64_t(n) * 4u, 4))))
    g = gemv_geometry(*d, k, n);
  if (g.fits) {
    hipFunction_t fn = is_gemv ? d->gemv_fast[f] : d->gemm_fast[f];
    return hipModuleLaunchKernel(fn, g.grid, is_gemv ? 1u : grid_y, 1, g.block, 1, 1, g.lds, stream, args, nullptr);
  }
  hipFunction_t fn = is_gemv ? d->gemv_generic[f] : d->gemm_generic[f];
  const uint32_t block = 256, rows_per_block = block / 64;
  const uint32_t grid = std::min<uint32_t>((n + rows_per_block - 1) / rows_per_block, uint32_t(d->cu_count) * 32u);
  return hipModuleLaunchKernel(fn, grid, is_gemv ? 1u : grid_y, 1, block, 1, 1, 0, stream, args, nullptr);
}

hipError_t launch_dequant(Fmt f, hipStream_t stream, uint64_t out, uint64_t w, uint64_t n_sb, int policy) {
  if (policy != 0 && policy != 1) return hipErrorInvalidValue;
  if (n_sb == 0) return hipSuccess;
  if (out == 0 || w == 0) return hipErrorInvalidValue;
  DeviceKernels* d = nullptr;
  hipError_t e = device_kernels(&d);
  if (e != hipSuccess) return e;
  const bool fast = policy == 0 && aligned(out, 16) && aligned(w, f == Q6K ? 2 : 16);
  const uint64_t threads = fast ? n_sb * 4 : n_sb * 256;
  const uint32_t grid = uint32_t(std::min<uint64_t>((threads + 255) / 256, uint64_t(d->cu_count) * 64u));
  if (fast) {
    void* args[] = {&out, &w, &n_sb};
    return hipModuleLaunchKernel(d->dequant_fast[f], grid, 1, 1, 256, 1, 1, 0, stream, args, nullptr);
  }
  void* args[] = {&out, &w, &n_sb, &policy};
  return hipModuleLaunchKernel(d->dequant_generic[f], grid, 1, 1, 256, 1, 1, 0, stream, args, nullptr);
}

}  // namespace

struct trn_ctx_s {
  int device;
};
struct trn_function_s {
  hipFunction_t fn;
  int kind;
  int fmt;
};
struct trn_module_s {
  hipModule_t module;
  bool builtin;
  std::mutex mutex;
  std::map<std::string, trn_function_s*> functions;
};
struct trn_event_s {
  hipEvent_t ev;
};

namespace {
trn_ctx_s g_ctx[kMaxDevices];
}

extern "C" {

// ---- 1/2. init and devices ---------------------------------------------------------------
trn_status trn_init(unsigned flags) { return st(hipInit(flags)); }

trn_status trn_device_get_count(int* count) {
  if (!count) return TRN_ERROR_INVALID_VALUE;
  *count = 0;
  return st(hipGetDeviceCount(count));
}

trn_status trn_device_get(trn_device* device, int ordinal) {
  if (!device) return TRN_ERROR_INVALID_VALUE;
  hipDevice_t d;
  TRN_TRY(hipDeviceGet(&d, ordinal));
  *device = static_cast<trn_device>(d);
  return TRN_SUCCESS;
}

trn_status trn_device_get_name(char* name, int len, trn_device device) {
  if (!name || len <= 0) return TRN_ERROR_INVALID_VALUE;
  return st(hipDeviceGetName(name, len, static_cast<hipDevice_t>(device)));
}

trn_status trn_device_total_mem(size_t* bytes, trn_device device) {
  if (!bytes) return TRN_ERROR_INVALID_VALUE;
  return st(hipDeviceTotalMem(bytes, static_cast<hipDevice_t>(device)));
}

// ---- 3. primary context -----------------------------------------------------------------
// HIP keeps one implicit primary context per device for the life of the process, so retain and
// release only validate the device; a context handle is the device it belongs to, and making it
// current selects that device for the calling thread.
trn_status trn_primary_ctx_retain(trn_ctx* ctx, trn_device device) {
  if (!ctx) return TRN_ERROR_INVALID_VALUE;
  int count = 0;
  TRN_TRY(hipGetDeviceCount(&count));
  if (device < 0 || device >= count || device >= kMaxDevices) return TRN_ERROR_INVALID_DEVICE;
  g_ctx[device].device = device;
  *ctx = &g_ctx[device];
  return TRN_SUCCESS;
}

trn_status trn_primary_ctx_release(trn_device device) {
  int count = 0;
  TRN_TRY(hipGetDeviceCount(&count));
  return device >= 0 && device < count ? TRN_SUCCESS : TRN_ERROR_INVALID_DEVICE;
}

trn_status trn_ctx_set_current(trn_ctx ctx) {
  if (!ctx) return TRN_ERROR_INVALID_VALUE;
  return st(hipSetDevice(ctx->device));
}

trn_status trn_ctx_synchronize(void) { return st(hipDeviceSynchronize()); }

// ---- 4. modules --------------------------------------------------------------------------
trn_status trn_module_load_data(trn_module* module, const void* image) {
  if (!module || !image) return TRN_ERROR_INVALID_VALUE;
  hipModule_t m = nullptr;
  TRN_TRY(hipModuleLoadData(&m, image));
  trn_module_s* h = new trn_module_s();
  h->module = m;
  h->builtin = false;
  *module = h;
  return TRN_SUCCESS;
}

trn_status trn_module_load_builtin(trn_module* module) {
  if (!module) return TRN_ERROR_INVALID_VALUE;
  hipModule_t m = nullptr;
  TRN_TRY(hipModuleLoadData(&m, trn_builtin_hsaco_begin));
  trn_module_s* h = new trn_module_s();
  h->module = m;
  h->builtin = true;
  *module = h;
  return TRN_SUCCESS;
}

trn_status trn_builtin_image(const void** image, size_t* size) {
  if (!image || !size) return TRN_ERROR_INVALID_VALUE;
  *image = trn_builtin_hsaco_begin;
  *size = size_t(trn_builtin_hsaco_end - trn_builtin_hsaco_begin);
  return TRN_SUCCESS;
}

trn_status trn_module_unload(trn_module module) {
  if (!module) return TRN_ERROR_INVALID_VALUE;
  hipError_t e = hipModuleUnload(module->module);
  for (auto& kv : module->functions) delete kv.second;
  delete module;
  return st(e);
}

trn_status trn_module_get_function(trn_function* func, trn_module module, const char* name) {
  if (!func || !module || !name) return TRN_ERROR_INVALID_VALUE;
  std::lock_guard<std::mutex> lock(module->mutex);
  auto it = module->functions.find(name);
  if (it != module->functions.end()) {
    *func = it->second;
    return TRN_SUCCESS;
  }
  hipFunction_t f = nullptr;
  TRN_TRY(hipModuleGetFunction(&f, module->module, name));
  trn_function_s* h = new trn_function_s{f, KIND_OTHER, 0};
  if (module->builtin) {
    const std::string n = name;
    for (int i = 0; i < NFMT; ++i) {
      if (n == std::string(kFmtName[i]) + "_gemv_warp_reduce") { h->kind = KIND_GEMV; h->fmt = i; }
      if (n == std::string(kFmtName[i]) + "_gemm_ggml") { h->kind = KIND_GEMM; h->fmt = i; }
    }
  }
  module->functions[name] = h;
  *func = h;
  return TRN_SUCCESS;
}

// ---- 5. memory ---------------------------------------------------------------------------
trn_status trn_mem_alloc(trn_dptr* ptr, size_t size) {
  if (!ptr) return TRN_ERROR_INVALID_VALUE;
  *ptr = 0;
  if (size == 0) return TRN_ERROR_INVALID_VALUE;  // cuMemAlloc rejects 0 bytes; callers skip the call
  void* p = nullptr;
  TRN_TRY(hipMalloc(&p, size));
  *ptr = reinterpret_cast<trn_dptr>(p);
  return TRN_SUCCESS;
}

trn_status trn_mem_free(trn_dptr ptr) {
  if (ptr == 0) return TRN_SUCCESS;
  return st(hipFree(reinterpret_cast<void*>(ptr)));
}

trn_status trn_memcpy_htod(trn_dptr dst, const void* src, size_t size) {
  if (size == 0) return TRN_SUCCESS;
  if (!dst || !src) return TRN_ERROR_INVALID_VALUE;
  return st(hipMemcpy(reinterpret_cast<void*>(dst), src, size, hipMemcpyHostToDevice));
}

trn_status trn_memcpy_dtoh(void* dst, trn_dptr src, size_t size) {
  if (size == 0) return TRN_SUCCESS;
  if (!dst || !src) return TRN_ERROR_INVALID_VALUE;
  return st(hipMemcpy(dst, reinterpret_cast<const void*>(src), size, hipMemcpyDeviceToHost));
}

trn_status trn_memcpy_htod_async(trn_dptr dst, const void* src, size_t size, trn_stream stream) {
  if (size == 0) return TRN_SUCCESS;
  if (!dst || !src) return TRN_ERROR_INVALID_VALUE;
  return st(hipMemcpyAsync(reinterpret_cast<void*>(dst), src, size, hipMemcpyHostToDevice, static_cast<hipStream_t>(stream)));
}

trn_status trn_memcpy_dtoh_async(void* dst, trn_dptr src, size_t size, trn_stream stream) {
  if (size == 0) return TRN_SUCCESS;
  if (!dst || !src) return TRN_ERROR_INVALID_VALUE;
  return st(hipMemcpyAsync(dst, reinterpret_cast<const void*>(src), size, hipMemcpyDeviceToHost, static_cast<hipStream_t>(stream)));
}

trn_status trn_memcpy_dtod(trn_dptr dst, trn_dptr src, size_t size) {
  if (size == 0) return TRN_SUCCESS;
  if (!dst || !src) return TRN_ERROR_INVALID_VALUE;
  return st(hipMemcpy(reinterpret_cast<void*>(dst), reinterpret_cast<const void*>(src), size, hipMemcpyDeviceToDevice));
}

trn_status trn_memcpy_dtod_async(trn_dptr dst, trn_dptr src, size_t size, trn_stream stream) {
  if (size == 0) return TRN_SUCCESS;
  if (!dst || !src) return TRN_ERROR_INVALID_VALUE;
  return st(hipMemcpyAsync(reinterpret_cast<void*>(dst), reinterpret_cast<const void*>(src), size, hipMemcpyDeviceToDevice,
                           static_cast<hipStream_t>(stream)));
}

trn_status trn_mem_get_info(size_t* free_bytes, size_t* total_bytes) {
  if (!free_bytes || !total_bytes) return TRN_ERROR_INVALID_VALUE;
  return st(hipMemGetInfo(free_bytes, total_bytes));
}

// ---- 6. streams and launch ---------------------------------------------------------------
trn_status trn_stream_create(trn_stream* stream, unsigned flags) {
  if (!stream) return TRN_ERROR_INVALID_VALUE;
  hipStream_t s = nullptr;
  TRN_TRY(hipStreamCreateWithFlags(&s, flags & TRN_STREAM_NON_BLOCKING ? hipStreamNonBlocking : hipStreamDefault));
  *stream = s;
  return TRN_SUCCESS;
}

trn_status trn_stream_destroy(trn_stream stream) {
  if (!stream) return TRN_ERROR_INVALID_VALUE;
  return st(hipStreamDestroy(static_cast<hipStream_t>(stream)));
}

trn_status trn_stream_synchronize(trn_stream stream) { return st(hipStreamSynchronize(static_cast<hipStream_t>(stream))); }

trn_status trn_launch_kernel(trn_function func, unsigned grid_x, unsigned grid_y, unsigned grid_z, unsigned block_x,
                             unsigned block_y, unsigned block_z, unsigned shared_mem_bytes, trn_stream stream,
                             void** kernel_params, void** extra) {
  if (!func) return TRN_ERROR_INVALID_VALUE;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (func->kind == KIND_GEMV || func->kind == KIND_GEMM) {
    if (!kernel_params) return TRN_ERROR_INVALID_VALUE;  // the `extra` buffer form is not used by the reference
    for (int i = 0; i < (func->kind == KIND_GEMV ? 5 : 6); ++i)
      if (!kernel_params[i]) return TRN_ERROR_INVALID_VALUE;
    uint64_t p0, p1, p2;
    std::memcpy(&p0, kernel_params[0], 8);
    std::memcpy(&p1, kernel_params[1], 8);
    std::memcpy(&p2, kernel_params[2], 8);
    if (func->kind == KIND_GEMV) {  // (y, w, x, k_dim, n_dim)
      uint32_t k, n;
      std::memcpy(&k, kernel_params[3], 4);
      std::memcpy(&n, kernel_params[4], 4);
      return st(launch_gemm_like(Fmt(func->fmt), s, p2, p1, p0, 1, n, k, true));
    }
    uint32_t m, n, k;  // (a, b_quant, c, m, n, k)
    std::memcpy(&m, kernel_params[3], 4);
    std::memcpy(&n, kernel_params[4], 4);
    std::memcpy(&k, kernel_params[5], 4);
    return st(launch_gemm_like(Fmt(func->fmt), s, p0, p1, p2, m, n, k, false));
  }
  return st(hipModuleLaunchKernel(func->fn, grid_x, grid_y, grid_z, block_x, block_y, block_z, shared_mem_bytes, s,
                                  kernel_params, extra));
}

// ---- 8. typed launchers ------------------------------------------------------------------
trn_status trn_q4k_gemv(trn_stream s, trn_dptr y, trn_dptr w, trn_dptr x, uint32_t k, uint32_t n) {
  return st(launch_gemm_like(Q4K, static_cast<hipStream_t>(s), x, w, y, 1, n, k, true));
}
trn_status trn_q5k_gemv(trn_stream s, trn_dptr y, trn_dptr w, trn_dptr x, uint32_t k, uint32_t n) {
  return st(launch_gemm_like(Q5K, static_cast<hipStream_t>(s), x, w, y, 1, n, k, true));
}
trn_status trn_q6k_gemv(trn_stream s, trn_dptr y, trn_dptr w, trn_dptr x, uint32_t k, uint32_t n) {
  return st(launch_gemm_like(Q6K, static_cast<hipStream_t>(s), x, w, y, 1, n, k, true));
}
trn_status trn_q4k_gemm(trn_stream s, trn_dptr a, trn_dptr b, trn_dptr c, uint32_t m, uint32_t n, uint32_t k) {
  return st(launch_gemm_like(Q4K, static_cast<hipStream_t>(s), a, b, c, m, n, k, false));
}
trn_status trn_q5k_gemm(trn_stream s, trn_dptr a, trn_dptr b, trn_dptr c, uint32_t m, uint32_t n, uint32_t k) {
  return st(launch_gemm_like(Q5K, static_cast<hipStream_t>(s), a, b, c, m, n, k, false));
}
trn_status trn_q6k_gemm(trn_stream s, trn_dptr a, trn_dptr b, trn_dptr c, uint32_t m, uint32_t n, uint32_t k) {
  return st(launch_gemm_like(Q6K, static_cast<hipStream_t>(s), a, b, c, m, n, k, false));
}

trn_status trn_kquant_gemv_batch(trn_stream s, const trn_gemv_desc* descs, uint32_t count) {
  if (count == 0) return TRN_SUCCESS;
  if (!descs) return TRN_ERROR_INVALID_VALUE;
  for (uint32_t i = 0; i < count; ++i)  // validate the whole list before anything is launched
    if (descs[i].fmt < 4 || descs[i].fmt > 6 || descs[i].reserved != 0 || descs[i].k % 256u != 0) return TRN_ERROR_INVALID_VALUE;
  for (uint32_t i = 0; i < count; ++i) {
    const trn_gemv_desc& d = descs[i];
    hipError_t e = launch_gemm_like(Fmt(d.fmt - 4), static_cast<hipStream_t>(s), d.x, d.w, d.y, 1, d.n, d.k, true);
    if (e != hipSuccess) return st(e);
  }
  return TRN_SUCCESS;
}

// ---- 9. dequantise test surface ----------------------------------------------------------
trn_status trn_q4k_dequant_f32(trn_stream s, trn_dptr out, trn_dptr w, uint64_t n_sb, int policy) {
  return st(launch_dequant(Q4K, static_cast<hipStream_t>(s), out, w, n_sb, policy));
}
trn_status trn_q5k_dequant_f32(trn_stream s, trn_dptr out, trn_dptr w, uint64_t n_sb, int policy) {
  return st(launch_dequant(Q5K, static_cast<hipStream_t>(s), out, w, n_sb, policy));
}
trn_status trn_q6k_dequant_f32(trn_stream s, trn_dptr out, trn_dptr w, uint64_t n_sb, int policy) {
  return st(launch_dequant(Q6K, static_cast<hipStream_t>(s), out, w, n_sb, policy));
}

// ---- 10. timing, errors, tuning ----------------------------------------------------------
trn_status trn_event_create(trn_event* event) {
  if (!event) return TRN_ERROR_INVALID_VALUE;
  hipEvent_t e = nullptr;
  TRN_TRY(hipEventCreate(&e));
  *event = new trn_event_s{e};
  return TRN_SUCCESS;
}

trn_status trn_event_destroy(trn_event event) {
  if (!event) return TRN_ERROR_INVALID_VALUE;
  hipError_t e = hipEventDestroy(event->ev);
  delete event;
  return st(e);
}

trn_status trn_event_record(trn_event event, trn_stream stream) {
  if (!event) return TRN_ERROR_INVALID_VALUE;
  return st(hipEventRecord(event->ev, static_cast<hipStream_t>(stream)));
}

trn_status trn_event_synchronize(trn_event event) {
  if (!event) return TRN_ERROR_INVALID_VALUE;
  return st(hipEventSynchronize(event->ev));
}

trn_status trn_event_elapsed_ms(float* ms, trn_event start, trn_event stop) {
  if (!ms || !start || !stop) return TRN_ERROR_INVALID_VALUE;
  return st(hipEventElapsedTime(ms, start->ev, stop->ev));
}

trn_status trn_copy_u128(trn_stream stream, trn_dptr dst, trn_dptr src, uint64_t bytes) {
  if (bytes % 16u != 0 || !aligned(dst, 16) || !aligned(src, 16)) return TRN_ERROR_INVALID_VALUE;
  if (bytes == 0) return TRN_SUCCESS;
  if (!dst || !src) return TRN_ERROR_INVALID_VALUE;
  DeviceKernels* d = nullptr;
  TRN_TRY(device_kernels(&d));
  uint64_t n = bytes / 16u;
  const uint32_t grid = uint32_t(std::min<uint64_t>((n + 255) / 256, uint64_t(d->cu_count) * 32u));
  void* args[] = {&dst, &src, &n};
  return st(hipModuleLaunchKernel(d->copy_u128, grid, 1, 1, 256, 1, 1, 0, static_cast<hipStream_t>(stream), args, nullptr));
}

const char* trn_error_name(trn_status status) { return hipGetErrorName(static_cast<hipError_t>(status)); }
const char* trn_error_string(trn_status status) { return hipGetErrorString(static_cast<hipError_t>(status)); }

trn_status trn_device_cu_count(int* count) {
  if (!count) return TRN_ERROR_INVALID_VALUE;
  int dev = 0;
  TRN_TRY(hipGetDevice(&dev));
  return st(hipDeviceGetAttribute(count, hipDeviceAttributeMultiprocessorCount, dev));
}

trn_status trn_set_tuning(const char* key, int value) {
  if (!key || value < 0) return TRN_ERROR_INVALID_VALUE;
  std::lock_guard<std::mutex> lock(g_mutex);
  if (!std::strcmp(key, "gemv_blocks_per_cu")) { g_tune_blocks_per_cu = value; return TRN_SUCCESS; }
  if (!std::strcmp(key, "gemv_row_groups")) { g_tune_row_groups = value; return TRN_SUCCESS; }
  return TRN_ERROR_INVALID_VALUE;
}

}  // extern "C"
