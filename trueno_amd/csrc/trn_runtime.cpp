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
#include <atomic>
#include <cstdlib>
#include <cstdio>
#include <cstring>
#include <map>
#include <mutex>
#include <string>
#include <tuple>
#include <utility>
#include <vector>

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

// trn_noalloc.hip: the library's static device scratch buffer (one copy per GPU)
extern "C" hipError_t trn_noalloc_scratch_setup(int dev);
extern "C" uint64_t trn_noalloc_scratch(int dev, size_t* bytes);

namespace {

enum Fmt { Q4K = 0, Q5K = 1, Q6K = 2, NFMT = 3 };
const char* const kFmtName[NFMT] = {"q4k", "q5k", "q6k"};
const uint32_t kSbBytes[NFMT] = {144, 176, 210};

// kinds of functions the launch-by-name path recognises
// KIND_OTHER: a function of a caller's own code object, launched exactly as given.  KIND_INTERNAL: a kernel of the
// built-in code object that is not one of the reference's names; its geometry and extra arguments belong to the
// typed entry points, so a by-name launch of it is refused.
enum Kind { KIND_OTHER = 0, KIND_GEMV = 1, KIND_GEMM = 2, KIND_GEMM_SIMPLIFIED = 3, KIND_RESIDUAL_ADD = 4, KIND_SWIGLU = 5,
            KIND_RMSNORM = 6, KIND_RESIDUAL_RMSNORM = 7, KIND_GEMV_F32 = 8, KIND_ATTENTION = 9, KIND_INTERNAL = 10 };

constexpr int kMaxDevices = 64;
#ifndef KQ_U
#define KQ_U 2
#endif
constexpr uint32_t kGemvRowsPerBatch = KQ_U;  // U of the fast GEMV kernel (the build passes it to both sides)
constexpr uint32_t kGemvMaxWaves = 12;        // __launch_bounds__(768) of the fast GEMV kernels
constexpr uint32_t kFastLdsLimit = 64 * 1024;  // dynamic LDS the fast kernels may ask for
constexpr uint32_t kLdsScratch = 64 + 256;     // group sums of squares (k/256 <= 64 floats) at the end of the fast kernels' LDS
// The engine for matrices of one slab (k <= 4096) streams the rows through LDS (chain_step_stream of kquant_chain.hip.h):
// behind the vector, the partial sums and the scratch every wave owns a ring of two slots of this many bytes (a batch of
// KQ_U rows of 16 blocks as they lie in LDS - a Q6_K block takes 224 bytes there - in whole KB: StreamSlot of the kernels).
constexpr uint32_t kChainStreamFlag = 16u;     // CHAIN_STREAM_LDS
constexpr uint32_t kStreamLdsLimit = 160 * 1024 - 1024;   // dynamic LDS such a launch may ask for (the CU has 160 KB; static LDS is a few words)
constexpr uint32_t stream_slot_bytes(uint32_t sb_bytes) { return (kGemvRowsPerBatch * 16u * (sb_bytes == 210u ? 224u : sb_bytes) + 1023u) / 1024u * 1024u; }

struct DeviceKernels {
  bool loaded = false;
  hipModule_t module = nullptr;
  int cu_count = 0;
  hipFunction_t gemv_fast[NFMT] = {}, gemv_flags[NFMT] = {}, gemv_generic[NFMT] = {};
  hipFunction_t fill_u32 = nullptr, gemv_group = nullptr, gemv_many = nullptr, phases = nullptr;
  int cooperative = 0;
  uint32_t resident_small = 3;   // resident 256-thread GEMV workgroups per CU (occupancy of the one-slab geometry)
  hipFunction_t gemm_fast[NFMT] = {}, gemm_generic[NFMT] = {}, gemm_as_written[NFMT] = {};
  hipFunction_t dequant_fast[NFMT] = {}, dequant_generic[NFMT] = {};
  hipFunction_t copy_u128 = nullptr, read_u128 = nullptr;
  hipFunction_t residual_add = nullptr, swiglu = nullptr, rmsnorm = nullptr, residual_rmsnorm = nullptr;
  hipFunction_t gemv_f32_fast = nullptr, gemv_f32_generic = nullptr, q5k_from_ggml = nullptr, attention = nullptr;
  hipFunction_t gemm_f16[NFMT][2] = {};   // [format][4 or 8 strips per workgroup]
  hipFunction_t gemm_f16_w12 = nullptr;   // Q4_K: 12 strips per workgroup
  hipFunction_t gemm_f16_t2[2] = {};      // Q4_K, Q5_K: 8 strips and two token tiles per workgroup
  hipFunction_t gemm_few[2] = {};         // Q4_K, integer matrix cores, built for 2 and 4 tokens
  hipFunction_t gemm_simplified = nullptr, dequant_simplified = nullptr;
};

std::mutex g_mutex;
// The tuning knobs are process-wide and meant for tests and measurements: atomics, so that a thread that flips one
// while another launches is a race on the setting, never on memory.
DeviceKernels g_dev[kMaxDevices];
std::atomic<int> g_tune_epoch{0};           // counts the calls of trn_set_tuning: plans made under other settings are stale
std::atomic<int> g_tune_blocks_per_cu{0};
std::atomic<int> g_tune_row_groups{0};
std::atomic<int> g_tune_batch_mode{0};   // 0: launches (default); 1: resident phases + barriers
std::atomic<int> g_tune_chain_spin_limit{0};
std::atomic<int> g_tune_group_off{0};
std::atomic<int> g_tune_group_pool_off{0};
std::atomic<int> g_tune_group_pool_waves{0};  // 1: grouped launches cut every entry's rows evenly (no run-time pools)
std::atomic<int> g_tune_gemm_mfma_off{0};   // 1: the Q4_K GEMM never takes the matrix-core form
std::atomic<int> g_tune_gemm_tiles{0};      // token tiles per workgroup of the matrix-core GEMM: 0 by the rule, 1, 2
std::atomic<int> g_tune_gemm_ksplit{0};     // parts of K in the matrix-core GEMM (0: chosen from the shape)
std::atomic<int> g_tune_attention_min_steps{0};
std::atomic<int> g_tune_group_window{0};       // entries of a list a launch may look ahead over (0: twice the most it may hold)
std::atomic<int> g_tune_group_waves{0};        // least waves per workgroup of a launch of up to sixteen entries (0: 8, or what the widest entry needs)
std::atomic<int> g_tune_group_max{0};          // most entries in one launch (0: as many as the list offers, up to kManyMax)
std::atomic<int> g_tune_slab_weight{0};        // percent a launch adds to an entry's bytes per slab of 4096 columns beyond the first (0: 40)
std::atomic<int> g_tune_attention_per_cu{0};   // workgroups per CU the single-query attention aims at (0: default)
std::atomic<int> g_tune_gemm_waves{0};      // strips of 32 rows per workgroup of the matrix-core GEMM: 4, 8 or (Q4_K) 12 (0: default)
std::atomic<int> g_tune_stream_off{0};      // 1: one-slab GEMVs load their rows into registers straight from memory (no LDS ring)
std::atomic<int> g_tune_stream_q6k{0};      // 1: Q6_K one-slab GEMVs stream through LDS too
std::atomic<int> g_tune_stream_cost{0};     // percent of its bytes a streamed entry counts for when a grouped launch shares out its workgroups (0: default)
std::atomic<int> g_tune_stream_min_rows{0}; // a single GEMV streams when a wave gets at least this many rows (0: default)
std::atomic<int> g_tune_many_waves{0};      // waves per workgroup of a launch of more than sixteen entries (0: 12)
std::atomic<int> g_tune_group_stream_min_rows{0};  // an entry of a launch of up to sixteen streams when a wave gets at least this many rows (0: default)
std::atomic<int> g_tune_many_item_kb{0};    // what a further piece of work costs a workgroup of such a launch, in KB of weights (0: default)
std::atomic<int> g_tune_many_slab_weight{0};  // percent such a launch adds to an entry's bytes per slab of 4096 columns beyond the first (0: default)
std::atomic<int> g_tune_stream_waves{0};    // waves per workgroup of a single streamed GEMV (0: default)
std::atomic<int> g_tune_gemm_few{0};        // the integer matrix-core kernel for two to four tokens: 0 by the rule, 1 wherever it can run, 2 never

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
          (e = get_fn(m, &t.gemv_flags[f], p + "_gemv_flags")) != hipSuccess ||
          (e = get_fn(m, &t.gemv_generic[f], p + "_gemv_generic")) != hipSuccess ||
          (e = get_fn(m, &t.gemm_fast[f], p + "_gemm_ggml")) != hipSuccess ||
          (e = get_fn(m, &t.gemm_generic[f], p + "_gemm_generic")) != hipSuccess ||
          (e = get_fn(m, &t.gemm_as_written[f], p + "_gemm_as_written")) != hipSuccess ||
          (e = get_fn(m, &t.dequant_fast[f], p + "_dequant_f32")) != hipSuccess ||
          (e = get_fn(m, &t.dequant_generic[f], p + "_dequant_f32_generic")) != hipSuccess) {
        (void)hipModuleUnload(m);
        return e;
      }
    }
    if ((e = get_fn(m, &t.copy_u128, "kq_copy_u128")) != hipSuccess ||
        (e = get_fn(m, &t.read_u128, "kq_read_u128")) != hipSuccess ||
        (e = get_fn(m, &t.gemv_f32_fast, "gemv_f32_fast")) != hipSuccess ||
        (e = get_fn(m, &t.q5k_from_ggml, "q5k_from_ggml")) != hipSuccess ||
        (e = get_fn(m, &t.attention, "incremental_attention")) != hipSuccess ||
        (e = get_fn(m, &t.gemv_f32_generic, "gemv_coalesced")) != hipSuccess ||
        (e = get_fn(m, &t.residual_add, "residual_add")) != hipSuccess ||
        (e = get_fn(m, &t.swiglu, "fused_swiglu")) != hipSuccess ||
        (e = get_fn(m, &t.rmsnorm, "rmsnorm")) != hipSuccess ||
        (e = get_fn(m, &t.residual_rmsnorm, "fused_residual_rmsnorm")) != hipSuccess ||
        (e = get_fn(m, &t.gemv_group, "kq_gemv_group")) != hipSuccess ||
        (e = get_fn(m, &t.gemv_many, "kq_gemv_many")) != hipSuccess ||
        (e = get_fn(m, &t.phases, "kq_gemv_phases")) != hipSuccess ||
        (e = get_fn(m, &t.gemm_simplified, "q4k_gemm_fused")) != hipSuccess ||
        (e = get_fn(m, &t.dequant_simplified, "q4k_simplified_dequant_f32")) != hipSuccess ||
        (e = get_fn(m, &t.gemm_f16[0][0], "q4k_gemm_f16_w4")) != hipSuccess ||
        (e = get_fn(m, &t.gemm_f16[0][1], "q4k_gemm_f16_w8")) != hipSuccess ||
        (e = get_fn(m, &t.gemm_f16[1][0], "q5k_gemm_f16_w4")) != hipSuccess ||
        (e = get_fn(m, &t.gemm_f16[1][1], "q5k_gemm_f16_w8")) != hipSuccess ||
        (e = get_fn(m, &t.gemm_f16_t2[0], "q4k_gemm_f16_w8t2")) != hipSuccess ||
        (e = get_fn(m, &t.gemm_f16_w12, "q4k_gemm_f16_w12")) != hipSuccess ||
        (e = get_fn(m, &t.gemm_f16_t2[1], "q5k_gemm_f16_w8t2")) != hipSuccess ||
        (e = get_fn(m, &t.gemm_f16[2][0], "q6k_gemm_f16_w4")) != hipSuccess ||
        (e = get_fn(m, &t.gemm_f16[2][1], "q6k_gemm_f16_w8")) != hipSuccess ||
        (e = get_fn(m, &t.gemm_few[0], "q4k_gemm_few_t2")) != hipSuccess ||
        (e = get_fn(m, &t.gemm_few[1], "q4k_gemm_few_t4")) != hipSuccess ||
        (e = get_fn(m, &t.fill_u32, "kq_fill_u32")) != hipSuccess) {
      (void)hipModuleUnload(m);
      return e;
    }
    if ((e = hipDeviceGetAttribute(&t.cu_count, hipDeviceAttributeMultiprocessorCount, dev)) != hipSuccess) {
      (void)hipModuleUnload(m);
      return e;
    }
    if (t.cu_count <= 0) t.cu_count = 256;
    (void)hipDeviceGetAttribute(&t.cooperative, hipDeviceAttributeCooperativeLaunch, dev);
    int occ = 0;
    if (hipModuleOccupancyMaxActiveBlocksPerMultiprocessor(&occ, t.gemv_group, 256, 4096 * 4 + 1024) == hipSuccess && occ >= 1)
      t.resident_small = uint32_t(std::min(occ, 4));
    // this GPU's copy of the static scratch buffer (trn_q4k_gemm_noalloc): found here, once, so that the entry point
    // itself never has to set anything up
    if ((e = trn_noalloc_scratch_setup(dev)) != hipSuccess) {
      (void)hipModuleUnload(m);
      return e;
    }
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

// Can an n x k matrix of this format go through the streamed engine?  (one slab; any alignment the fast kernels take)
// Q6_K stays on the register path by default: its slots are 7 KB (the 210-byte blocks re-spaced to 224), so a workgroup
// of twelve waves has no room for its rings, and a launch alone gains nothing (32000 x 4096: 19.2-20 us either way).  A
// long list of one-slab Q6_K matrices in workgroups of eight waves ("many_waves") is 4-7 % faster streamed (64 matrices
// of 4096 x 4096: 144 against 155 us; eight of 32000 x 4096: 138 against 147 us).  "gemv_stream_q6k" turns it on.
bool stream_ok(uint32_t fmt_code, uint32_t k, uint32_t n) {
  return !g_tune_stream_off && k != 0 && k <= 4096u && n >= kGemvRowsPerBatch && (fmt_code != 6u || g_tune_stream_q6k);
}

// Geometry of a single streamed GEMV: workgroups of `waves` waves, as many per CU as their LDS allows (two by default).
GemvGeometry stream_geometry(const DeviceKernels& d, Fmt f, uint32_t k, uint32_t n) {
  GemvGeometry g;
  const uint32_t waves = g_tune_stream_waves > 0 ? std::min<uint32_t>(uint32_t(g_tune_stream_waves), kGemvMaxWaves) : 4u;
  const uint32_t ring = waves * 2u * stream_slot_bytes(kSbBytes[f]);
  const uint64_t fixed = uint64_t(k) * 4u + kLdsScratch + ring;
  if (fixed + kGemvRowsPerBatch * 4u > kStreamLdsLimit) return g;
  const uint32_t fit = uint32_t(std::max<uint64_t>(1, (160u * 1024u) / (fixed + 1024u)));
  const uint32_t per_cu = g_tune_blocks_per_cu > 0 ? uint32_t(g_tune_blocks_per_cu) : std::min(fit, std::max(1u, 8u / waves));
  const uint64_t target_blocks = uint64_t(d.cu_count) * per_cu;
  const uint32_t ug = kGemvRowsPerBatch;
  uint64_t rows = (uint64_t(n) + target_blocks - 1) / target_blocks;
  rows = std::max<uint64_t>(ug, (rows + ug - 1) / ug * ug);
  const uint64_t max_rows = (kStreamLdsLimit - fixed) / 4u / ug * ug;
  rows = std::min<uint64_t>(rows, max_rows);
  // A wave that gets only a batch or two never reaches the steady state the ring is there for, and the start of a
  // streamed workgroup is the longer one (Q4_K 4096 x 4096 alone: 5.2 us on the register path, 6.4 us streamed).
  const uint32_t min_rows = g_tune_stream_min_rows > 0 ? uint32_t(g_tune_stream_min_rows) : 16u;
  if (rows < uint64_t(min_rows) * waves) return g;
  g.grid = uint32_t((uint64_t(n) + rows - 1) / rows);
  g.block = 64u * waves;
  g.lds = uint32_t(fixed + rows * 4u);
  g.fits = true;
  return g;
}

GemvGeometry gemv_geometry(const DeviceKernels& d, uint32_t k, uint32_t n, uint32_t max_waves = kGemvMaxWaves) {
  GemvGeometry g;
  const uint32_t nsb = k / 256u;
  const uint32_t slabs = (nsb + 15u) / 16u;
  const uint32_t sw = std::min<uint32_t>(slabs, max_waves);
  // Measured on MI355X: one slab (k <= 4096) runs best as workgroups of 4 waves, as many as are resident; with
  // several slabs every workgroup stages the whole (large) activation vector, so one big workgroup per CU wins
  // (12 waves: what the kernels' registers let a CU hold).
  uint32_t groups = g_tune_row_groups > 0 ? uint32_t(g_tune_row_groups) : (sw == 1 ? 4u : max_waves / sw);
  groups = std::max<uint32_t>(1u, std::min<uint32_t>(groups, max_waves / sw));
  const uint32_t ug = kGemvRowsPerBatch * groups;
  // one-slab kernels: as many workgroups as are resident at once (3 per CU at the kernels' register use; a
  // fourth per CU would only start when one of the first three has finished)
  const uint32_t per_cu = g_tune_blocks_per_cu > 0 ? uint32_t(g_tune_blocks_per_cu) : (sw == 1 ? d.resident_small : 1u);
  const uint64_t target_blocks = uint64_t(d.cu_count) * per_cu;
  uint64_t rows = (uint64_t(n) + target_blocks - 1) / target_blocks;
  rows = std::max<uint64_t>(ug, (rows + ug - 1) / ug * ug);
  // keep activations + partial sums within the LDS the kernel may ask for
  const uint64_t x_bytes = uint64_t(k) * 4u;
  if (x_bytes + uint64_t(sw) * ug * 4u + kLdsScratch > kFastLdsLimit) return g;
  const uint64_t max_rows = (kFastLdsLimit - kLdsScratch - x_bytes) / (uint64_t(sw) * 4u) / ug * ug;
  rows = std::min<uint64_t>(rows, max_rows);
  g.grid = uint32_t((uint64_t(n) + rows - 1) / rows);
  // the kernel recomputes rows-per-block from the grid; it can only come out <= rows
  g.block = 64u * sw * groups;
  g.lds = uint32_t(x_bytes + uint64_t(sw) * rows * 4u + kLdsScratch);
  g.fits = true;
  return g;
}

bool aligned(uint64_t p, uint64_t a) { return (p & (a - 1)) == 0; }

bool gemv_fast_ok(Fmt f, uint64_t y, uint64_t w, uint64_t x) {
  // 128-bit activation loads; Q4_K/Q5_K blocks are streamed with aligned 128-bit loads (their
  // rows are multiples of 16 bytes); Q6_K blocks (210 bytes) only need their natural 2 bytes.
  return aligned(x, 16) && aligned(y, 4) && aligned(w, f == Q6K ? 2 : 16);
}

// Element-wise steps of a decoder layer (decode_glue.hip.h).  kind: KIND_RESIDUAL_ADD or KIND_SWIGLU.
hipError_t launch_elementwise(Kind kind, hipStream_t stream, uint64_t a, uint64_t b, uint64_t out, uint32_t n) {
  if (n == 0) return hipSuccess;
  if (!a || !b || !out || !aligned(a, 4) || !aligned(b, 4) || !aligned(out, 4)) return hipErrorInvalidValue;
  DeviceKernels* d = nullptr;
  hipError_t e = device_kernels(&d);
  if (e != hipSuccess) return e;
  const uint32_t grid = std::max(1u, std::min((n + 255u) / 256u, uint32_t(d->cu_count) * 8u));
  void* args[] = {&a, &b, &out, &n};
  return hipModuleLaunchKernel(kind == KIND_SWIGLU ? d->swiglu : d->residual_add, grid, 1, 1, 256, 1, 1, 0, stream, args, nullptr);
}

// residual == 0: rmsnorm; else fused_residual_rmsnorm.  One row, one workgroup.
hipError_t launch_rmsnorm(hipStream_t stream, uint64_t residual, uint64_t in, uint64_t out, uint64_t gamma, uint32_t hidden,
                          float eps, bool with_residual) {
  if (hidden == 0) return hipSuccess;
  if (!in || !out || !gamma || (with_residual && !residual) || !aligned(in, 4) || !aligned(out, 4) || !aligned(gamma, 4) ||
      !aligned(residual, 4))
    return hipErrorInvalidValue;
  DeviceKernels* d = nullptr;
  hipError_t e = device_kernels(&d);
  if (e != hipSuccess) return e;
  const uint32_t block = hidden <= 256u ? 64u : hidden <= 2048u ? 256u : 1024u;
  if (with_residual) {
    void* args[] = {&residual, &in, &out, &gamma, &hidden, &eps};
    return hipModuleLaunchKernel(d->residual_rmsnorm, 1, 1, 1, block, 1, 1, 0, stream, args, nullptr);
  }
  void* args[] = {&in, &out, &gamma, &hidden, &eps};
  return hipModuleLaunchKernel(d->rmsnorm, 1, 1, 1, block, 1, 1, 0, stream, args, nullptr);
}

// Per-(device, stream) scratch buffers of the kernels that cut their work in parts (partial results + arrival
// counters at the front).  g_ws_mutex is held across lookup, growth and the launch that zeroes new counters, so two
// threads on two streams never see a half-grown buffer; a buffer only ever belongs to one stream, and work on one
// stream is ordered, so the kernels themselves need no lock.  New counters are zeroed by a small fill kernel, not by
// hipMemsetAsync: the call may be recorded into a HIP graph by a capturing caller.
struct ScratchWorkspace {
  void* buf = nullptr;
  size_t cap = 0;
};
using ScratchMap = std::map<std::pair<int, hipStream_t>, ScratchWorkspace>;
std::mutex g_ws_mutex;

hipError_t acquire_scratch(ScratchMap& map, DeviceKernels* d, hipStream_t stream, size_t need, size_t zero_bytes, uint64_t* base) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  std::lock_guard<std::mutex> lock(g_ws_mutex);
  ScratchWorkspace& ws = map[std::make_pair(dev, stream)];
  if (ws.cap < need) {
    if (ws.buf) {
      if ((e = hipStreamSynchronize(stream)) != hipSuccess) return e;   // work in flight may still use the old buffer
      (void)hipFree(ws.buf);
      ws.buf = nullptr;
      ws.cap = 0;
    }
    if ((e = hipMalloc(&ws.buf, need)) != hipSuccess) return e;
    ws.cap = need;
    uint32_t words = uint32_t(zero_bytes / 4u), zero = 0u;
    void* fill_args[] = {&ws.buf, &words, &zero};
    const uint32_t grid = std::max(1u, std::min(64u, (words + 255u) / 256u));
    if ((e = hipModuleLaunchKernel(d->fill_u32, grid, 1, 1, 256, 1, 1, 0, stream, fill_args, nullptr)) != hipSuccess) return e;
  }
  *base = reinterpret_cast<uint64_t>(ws.buf);
  return hipSuccess;
}

// f32 GEMV y = A^T-style product with A K x N row-major (gemv_f32.hip.h).  Partial results of the parts of K and
// the arrival counters live in a per-(device, stream) buffer like the GEMM's.
ScratchMap g_gemv_f32_ws;

hipError_t launch_gemv_f32(hipStream_t stream, uint64_t y, uint64_t a, uint64_t x, uint32_t k, uint32_t n) {
  if (n == 0) return hipSuccess;
  if (!y || (k != 0 && (!a || !x)) || !aligned(y, 4) || !aligned(a, 4) || !aligned(x, 4)) return hipErrorInvalidValue;
  DeviceKernels* d = nullptr;
  hipError_t e = device_kernels(&d);
  if (e != hipSuccess) return e;
  if (k == 0 || n % 4u != 0 || !aligned(a, 16) || !aligned(y, 16)) {
    void* args[] = {&y, &a, &x, &k, &n};
    return hipModuleLaunchKernel(d->gemv_f32_generic, (n + 255u) / 256u, 1, 1, 256, 1, 1, 0, stream, args, nullptr);
  }
  const uint32_t tiles = (n + 255u) / 256u;
  // parts of K: about two workgroups of 8 waves per CU, at least 64 rows (8 per wave) each
  uint32_t parts = std::max(1u, (2u * uint32_t(d->cu_count) + tiles / 2u) / tiles);
  parts = std::max(1u, std::min(parts, (k + 63u) / 64u));
  uint32_t rows_per_part = (k + parts - 1u) / parts;
  rows_per_part = (rows_per_part + 7u) / 8u * 8u;
  parts = (k + rows_per_part - 1u) / rows_per_part;
  const size_t cnt_cap = 64u * 1024u, need = cnt_cap + (parts > 1u ? size_t(parts) * n * 4u : 0u);
  if (size_t(tiles) * 4u > cnt_cap) return hipErrorInvalidValue;
  uint64_t cnt = 0;
  if ((e = acquire_scratch(g_gemv_f32_ws, d, stream, need, cnt_cap, &cnt)) != hipSuccess) return e;   // the kernel leaves the counters at zero
  uint64_t part = cnt + cnt_cap;
  void* args[] = {&y, &a, &x, &part, &cnt, &k, &n, &rows_per_part, &parts};
  return hipModuleLaunchKernel(d->gemv_f32_fast, tiles * parts, 1, 1, 512, 1, 1, 0, stream, args, nullptr);
}

// Single-query attention over the KV cache (decode_attention.hip.h).  Per (device, stream): arrival counters per
// head and the chunks' partial softmax states.
ScratchMap g_attention_ws;

hipError_t launch_attention(hipStream_t stream, uint64_t q, uint64_t k, uint64_t v, uint64_t out, uint32_t seq_len,
                            uint32_t head_dim, uint32_t num_heads, uint32_t num_kv_heads, uint32_t max_seq_len, float scale) {
  if (num_heads == 0) return hipSuccess;
  if (!q || !k || !v || !out || seq_len == 0 || seq_len > max_seq_len || head_dim == 0 || head_dim % 4u != 0 || head_dim > 256u ||
      num_kv_heads == 0 || num_kv_heads > num_heads || num_heads > 16384u || !aligned(q, 16) || !aligned(k, 16) ||
      !aligned(v, 16) || !aligned(out, 16))
    return hipErrorInvalidValue;
  DeviceKernels* d = nullptr;
  hipError_t e = device_kernels(&d);
  if (e != hipSuccess) return e;
  uint32_t lpp_log2 = 0;
  while ((4u << lpp_log2) < head_dim) ++lpp_log2;
  const uint32_t lpp = 1u << lpp_log2, step = 4u * (64u >> lpp_log2);       // positions a workgroup takes at a time
  // chunks of positions per head: about two workgroups per CU, at least eight steps each (measured: 4 is 10 % slower at
  // 512 positions, more workgroups per CU are slower at every length)
  const uint32_t per_cu = g_tune_attention_per_cu > 0 ? uint32_t(g_tune_attention_per_cu) : 2u;
  uint32_t chunks = std::max(1u, (per_cu * uint32_t(d->cu_count) + num_heads - 1u) / num_heads);
  const uint32_t min_steps = g_tune_attention_min_steps > 0 ? uint32_t(g_tune_attention_min_steps) : 8u;
  chunks = std::max(1u, std::min(chunks, (seq_len + min_steps * step - 1u) / (min_steps * step)));
  uint32_t chunk = (seq_len + chunks - 1u) / chunks;
  chunk = (chunk + step - 1u) / step * step;
  chunks = (seq_len + chunk - 1u) / chunk;
  const size_t cnt_cap = 64u * 1024u, need = cnt_cap + (chunks > 1u ? size_t(num_heads) * chunks * lpp * 32u : 0u);
  uint64_t cnt = 0;
  if ((e = acquire_scratch(g_attention_ws, d, stream, need, cnt_cap, &cnt)) != hipSuccess) return e;   // the kernel leaves the counters at zero
  uint64_t part = cnt + cnt_cap;
  void* args[] = {&q, &k, &v, &out, &seq_len, &head_dim, &num_heads, &num_kv_heads, &max_seq_len, &scale, &lpp_log2, &chunk, &chunks,
                  &part, &cnt};
  return hipModuleLaunchKernel(d->attention, num_heads * chunks, 1, 1, 256, 1, 1, 0, stream, args, nullptr);
}

// Partial results and arrival counters of the matrix-core GEMM: one buffer per (device, stream), grown on
// demand and kept.  The counters are zero between products: the kernel puts them back.
ScratchMap g_gemm_ws;

constexpr uint32_t kGemmXpStageBytes = 16 * 1024 + 512 + 64;
constexpr size_t kGemmCounterBytes = size_t(1) << 16;   // arrival counters at the front of the GEMM's scratch buffer

// How a product on the matrix cores is cut: `waves` strips of 32 rows and nt token tiles of 16 per workgroup (groups of
// strips, tgroups of tiles), K in kparts parts of ksb super-blocks, so that the workgroups are about as many as the CUs.
struct GemmCut { uint32_t waves, nt, groups, tgroups, kparts, ksb; double us; };

// The cut with the least estimated time among: 8 strips and one tile, 8 strips and two tiles (Q4_K and Q5_K: the weight
// operands are built once for both; the Q6_K kernel has no registers left for it), 4 strips and one tile, 12 strips and
// one tile (Q4_K), each with the number of parts of K that estimates fastest.  Times in microseconds fitted to
// measurements on MI355X (Q4_K, 1024 x 4096 .. 32000 x 4096 and 4096 x 14336, 2 .. 512 tokens; they hold within about
// 15 %): 4 to the first super-block and for the stores (3.5 with 4 strips); a super-block takes a workgroup 2.0 (8 strips),
// 3.2 (8 strips, two tiles), 1.5 (4 strips) or 2.6 (12 strips; 2.4 alone on its CU, but with every CU busy the memory
// system gives the larger workgroups no more than the smaller), and no cut streams the weights faster than about
// 5 TB/s; with K in parts 2.5 for publishing a part, plus the time in which the workgroup that arrives last reads every
// part of its rows through one CU, at about 40 GB/s - with 16 parts of 8 strips that read alone took 6.5 us of 15
// (4096 x 4096, M = 16: 15.0 us with 8 strips, 10.3 us with 4).
// Examples (us, 8 strips, one tile and as many parts as fill the CUs -> chosen): 4096 x 4096 M = 16 15.0 -> 10.3;
// 1024 x 4096 M = 64 14.6 -> 9.8; 14336 x 4096 M = 48 41 -> 32, M = 128 65 -> 53, M = 512 234 -> 201; 4096 x 4096 M = 32 with
// two tiles would be 22.4 against 13; 11008 x 4096 (43 groups of 8 strips: six parts of K make 258 workgroups, two more
// than there are CUs) M = 4 19.5 -> 13.7 with four parts, M = 32 29.9 -> 18.7 with 12 strips (29 groups, eight parts).
// part_cap: the most bytes of partial sums the caller has room for; cuts that need more are left out (us = kCutDoesNotFit
// when none fits).
constexpr double kCutDoesNotFit = 1e30;
size_t gemm_part_bytes(uint32_t kparts, uint32_t tiles, uint32_t groups, uint32_t waves) {
  // per part of K, token tile and strip of 32 rows: 64 lanes x 8 sums
  return kparts > 1u ? (size_t(kparts) * tiles * groups * waves * 2048u + 255u) & ~size_t(255) : 0u;
}
GemmCut gemm_cut(const DeviceKernels& d, Fmt f, uint32_t m, uint32_t n, uint32_t k, size_t part_cap = ~size_t(0)) {
  const uint32_t nsb = k / 256u, tiles = (m + 15u) / 16u;
  const double weight_us = double(n) * nsb * kSbBytes[f] / 5.0e6;      // the weights once at 5 TB/s: no cut is faster
  auto cut_with = [&](uint32_t waves, uint32_t nt, uint32_t kparts) {
    GemmCut c{waves, nt, (n + 32u * waves - 1u) / (32u * waves), (tiles + nt - 1u) / nt, 1u, nsb, 0.0};
    const uint64_t units = uint64_t(c.groups) * c.tgroups;
    c.kparts = std::min(std::max(kparts, 1u), nsb);
    c.ksb = (nsb + c.kparts - 1u) / c.kparts;
    c.kparts = (nsb + c.ksb - 1u) / c.ksb;
    const uint64_t rounds = (units * c.kparts + uint64_t(d.cu_count) - 1u) / uint64_t(d.cu_count);
    const double step = waves == 4u ? 1.5 : waves == 12u ? 2.6 : nt == 2u ? 3.2 : 2.0;
    const double last_kb = double(c.kparts) * waves * nt * (m > 8u ? 2.0 : 1.0);
    c.us = (waves == 4u ? 3.5 : 4.0) + std::max(double(rounds) * c.ksb * step, weight_us) +
           (c.kparts > 1u ? 2.5 + last_kb / 40.0 : 0.0);
    if (gemm_part_bytes(c.kparts, tiles, c.groups, waves) > part_cap) c.us = kCutDoesNotFit;
    return c;
  };
  // the parts of K: as many as bring the workgroups to about the number of CUs, or fewer where that estimates faster (one
  // workgroup more than there are CUs costs a whole second round)
  auto cut_for = [&](uint32_t waves, uint32_t nt) {
    const uint64_t units = uint64_t((n + 32u * waves - 1u) / (32u * waves)) * ((tiles + nt - 1u) / nt);
    if (g_tune_gemm_ksplit > 0) return cut_with(waves, nt, uint32_t(g_tune_gemm_ksplit));
    const uint32_t most = uint32_t(std::min<uint64_t>((uint64_t(d.cu_count) + units / 2u) / units, nsb));
    GemmCut best = cut_with(waves, nt, most);
    for (uint32_t kp = most; kp-- > 1u;) {
      const GemmCut c = cut_with(waves, nt, kp);
      if (c.us < best.us) best = c;
    }
    return best;
  };
  const int tw = g_tune_gemm_waves, tt = g_tune_gemm_tiles;
  const bool twelve_ok = f == Q4K;      // (the other formats' weight tiles do not fit twelve times two into LDS)
  GemmCut best = cut_for(tw == 4 ? 4u : tw == 12 && twelve_ok ? 12u : 8u, 1u);
  if (tw == 0 && tt != 2) {
    const GemmCut four = cut_for(4u, 1u);
    if (four.us < best.us) best = four;
    if (twelve_ok) {
      const GemmCut twelve = cut_for(12u, 1u);
      if (twelve.us < best.us) best = twelve;
    }
  }
  if (tw != 4 && tw != 12 && f != Q6K && tiles >= 2u && tt != 1) {
    const GemmCut two = cut_for(8u, 2u);
    if (tt == 2 || two.us < best.us) best = two;
  }
  return best;
}

// ext_base != 0: the caller brings the scratch buffer (ext_cap bytes, counters at its front already zero); nothing is
// allocated and a product that needs more is refused.
hipError_t launch_kq_gemm_f16(DeviceKernels* d, Fmt f, hipStream_t stream, uint64_t a, uint64_t w, uint64_t c, uint32_t m,
                              uint32_t n, uint32_t k, uint64_t ext_base = 0, size_t ext_cap = 0, const GemmCut* given = nullptr) {
  const uint32_t nsb = k / 256u, tiles = (m + 15u) / 16u;
  const uint32_t kGemmWTileBytes = 32u * kSbBytes[f];
  // Q6_K: one weight tile per wave, rows 240 bytes apart (q6k_lds_bytes of the kernel's header)
  const uint32_t kGemmQ6TileBytes = 32u * 240u;
  // a caller's own scratch buffer: only cuts whose partial sums fit behind the counters
  const size_t part_cap = ext_base == 0 ? ~size_t(0) : ext_cap > kGemmCounterBytes ? ext_cap - kGemmCounterBytes : 0u;
  const GemmCut cut = given ? *given : gemm_cut(*d, f, m, n, k, part_cap);
  const uint32_t waves = cut.waves, nt = cut.nt, groups = cut.groups, tgroups = cut.tgroups, kparts = cut.kparts, ksb = cut.ksb;
  const uint32_t lds = f == Q6K ? 2u * kGemmXpStageBytes + waves * kGemmQ6TileBytes + 16u
                                : 2u * nt * kGemmXpStageBytes + 2u * waves * kGemmWTileBytes + 16u;
  // with several parts of K: one arrival counter per (group of strips, token tile)
  const size_t cnt_bytes = kparts > 1u ? size_t(groups) * tgroups * 4u : 0u;
  const size_t part_bytes = gemm_part_bytes(kparts, tiles, groups, waves);
  // the counters sit at the front of a region that only grows, so a larger product finds zeros there too (the
  // kernel puts every counter it used back to zero)
  const size_t cnt_cap = kGemmCounterBytes, need = cnt_cap + part_bytes;
  // (the kernel addresses the parts with 32-bit offsets; a cut by the estimate stays far below that, a forced one may not)
  if (cnt_bytes > cnt_cap || part_bytes >= (size_t(1) << 32)) return hipErrorInvalidValue;
  uint64_t cnt = ext_base;
  if (ext_base != 0) {
    if (need > ext_cap) return hipErrorInvalidValue;
  } else {
    hipError_t e = acquire_scratch(g_gemm_ws, d, stream, need, cnt_cap, &cnt);
    if (e != hipSuccess) return e;
  }
  const uint64_t padded = (uint64_t(groups) * kparts + 7u) / 8u * 8u;
  if (ksb > 0xFFFFu || groups > 0xFFFFu || tiles > 0xFFFFu || padded * tgroups > 0x7FFFFFFFu) return hipErrorInvalidValue;
  uint32_t nsb_arg = nsb;
  uint64_t geom = uint64_t(ksb) | uint64_t(kparts) << 16 | uint64_t(groups) << 32 | uint64_t(tiles) << 48;
  void* margs[] = {&a, &w, &c, &cnt, &m, &n, &nsb_arg, &geom};
  hipFunction_t fn = nt == 2u ? d->gemm_f16_t2[f] : waves == 12u ? d->gemm_f16_w12 : d->gemm_f16[f][waves == 8u];
  return hipModuleLaunchKernel(fn, uint32_t(padded * tgroups), 1, 1, 64 * waves, 1, 1, lds, stream, margs, nullptr);
}

// does the matrix-core form take this product?  (weights 16-byte aligned; Q6_K, whose blocks are 210 bytes, 2-byte aligned)
bool q4k_gemm_f16_ok(uint64_t a, uint64_t w, uint64_t c, uint32_t m, uint32_t n, uint32_t k, Fmt f = Q4K) {
  return m >= 2 && k != 0 && !g_tune_gemm_mfma_off && aligned(a, 16) && aligned(w, f == Q6K ? 2 : 16) && aligned(c, 4) &&
         k / 256u <= 0xFFFFu && (n + 127u) / 128u <= 0xFFFFu && (m + 15u) / 16u <= 0xFFFFu &&      // 16-bit fields of its geometry
         uint64_t((n + 127u) / 128u) * ((m + 15u) / 16u) <= 0x0FFFFFFFu;                            // its grid
}

// A few tokens against a small matrix are faster through the GEMV engine, one pass per token with the weights of the
// second and later passes coming from the caches, than through the matrix-core kernel with its start-up and its sum
// over the parts of K.  The engine's time in microseconds, fitted to measurements on MI355X (MB = weight bytes / 1e6):
// 3.9 + MB / 5.7 for the first token, MB / 5.8 + 0.15 for each further one (one slab of columns only; with k > 4096 a
// further pass costs as much as the first); the matrix cores' for up to 16 tokens, where the weights' bytes still
// count: 7.2 + MB / 4 with 4 strips per workgroup, 12 + MB / 9.4 with 8.
bool gemm_few_tokens_by_engine(const DeviceKernels& d, Fmt f, uint32_t m, uint32_t n, uint32_t k) {
  if (m > 8u || k > 4096u) return false;
  const double mb = double(n) * (k / 256u) * kSbBytes[f] / 1e6;
  const double matrix_cores = gemm_cut(d, f, m, n, k).waves == 4u ? 7.2 + mb / 4.0 : 12.0 + mb / 9.4;
  return 3.9 + mb / 5.7 + (m - 1u) * (mb / 5.8 + 0.15) < matrix_cores;
}

// The integer matrix-core kernel (kquant_few_i8.hip.h): Q4_K, two to four tokens, a row of W within one slab of 4096
// columns.  One workgroup per CU at most (its LDS), each with a run of rows that is a multiple of the tile's 32.
// Times in microseconds measured on MI355X (cold weights, k = 4096; n = 1024, 4096, 11008, 14336, 32000): two tokens
// 6.0, 6.2, 9.6, 10.3, 17.5; four tokens 8.4, 8.4, 11.7, 12.3, 20.0 - about 2.1 + 0.7 m (m = 2 or 4: what the kernel is
// built for) to make the digits and for the launch, and 4 per tile of 32 rows that a workgroup takes.  The other ways took, for two and four tokens, 4.9 / 5.1 (the
// GEMV engine, a pass per token), 7.2 / 9.2, 12.0 / 14.6, 14.8 / 14.8, 23.4 / 23.6 (the f16 matrix-core form).
constexpr uint32_t kFewRowPad = 32u;
double gemm_few_us(const DeviceKernels& d, uint32_t m, uint32_t n) {
  const uint32_t tiles = (n + 31u) / 32u, wgs = std::min<uint32_t>(tiles, uint32_t(d.cu_count));
  return 2.1 + 0.7 * (m <= 2u ? 2.0 : 4.0) + 4.0 * ((tiles + wgs - 1u) / wgs);
}
bool gemm_few_ok(Fmt f, uint64_t a, uint64_t w, uint64_t c, uint32_t m, uint32_t n, uint32_t k) {
  return f == Q4K && g_tune_gemm_few != 2 && m >= 2u && m <= 4u && k != 0 && k <= 4096u && n != 0 && aligned(a, 16) && aligned(w, 16) &&
         aligned(c, 4);
}
hipError_t launch_gemm_few(DeviceKernels* d, hipStream_t stream, uint64_t a, uint64_t w, uint64_t c, uint32_t m, uint32_t n, uint32_t k) {
  const uint32_t nsb = k / 256u, idx = m <= 2u ? 0u : 1u, ntok = 2u << idx;
  const uint32_t tiles = (n + 31u) / 32u, wgs = std::min<uint32_t>(tiles, uint32_t(d->cu_count));
  uint32_t rows_per_wg = (tiles + wgs - 1u) / wgs * 32u;
  const uint32_t grid = (n + rows_per_wg - 1u) / rows_per_wg;
  const uint32_t lds = 2u * 32u * (nsb * 144u + kFewRowPad) + 2u * 8u * 32u * ntok * 4u + ntok * nsb * 9u * 4u;   // lds_bytes of the kernel's header
  void* args[] = {&a, &w, &c, &m, &n, &k, &rows_per_wg};
  return hipModuleLaunchKernel(d->gemm_few[idx], grid, 1, 1, 512, 1, 1, lds, stream, args, nullptr);
}

constexpr double kBigAloneBytes = 64e6;      // from this size on a matrix alone takes the list kernel (launch_gemm_like, trn_kquant_gemv_batch)
bool list_groupable(DeviceKernels* dk, const trn_gemv_desc& d);
extern "C" {      // (defined further down inside the extern "C" part of the file: the same language linkage here)
hipError_t launch_gemv_group(DeviceKernels* d, hipStream_t stream, const trn_gemv_desc* descs, uint32_t len);
}

// Which kernel takes a product of m >= 1 tokens: the integer matrix cores (Q4_K, two to four tokens, where their fitted
// time is below the other ways'), the f16 matrix cores, or the GEMV engine with a pass per token (also: whatever the
// matrix-core forms cannot take).  A forced cut of the f16 form (tuning) takes that form.
enum class GemmRoute { kFew, kCores, kOther };
GemmRoute gemm_route(const DeviceKernels& d, Fmt f, uint64_t a, uint64_t w, uint64_t c, uint32_t m, uint32_t n, uint32_t k) {
  const bool cores_ok = q4k_gemm_f16_ok(a, w, c, m, n, k, f);
  const bool forced = g_tune_gemm_ksplit > 0 || g_tune_gemm_waves > 0 || g_tune_gemm_tiles > 0;
  if (gemm_few_ok(f, a, w, c, m, n, k) && (g_tune_gemm_few == 1 || !forced)) {
    const double mb = double(n) * (k / 256u) * kSbBytes[f] / 1e6;
    const double engine = 3.9 + mb / 5.7 + (m - 1u) * (mb / 5.8 + 0.15);      // (gemm_few_tokens_by_engine)
    const double cores = !cores_ok ? 1e30 : gemm_cut(d, f, m, n, k).waves == 4u ? 7.2 + mb / 4.0 : 12.0 + mb / 9.4;
    if (g_tune_gemm_few == 1 || gemm_few_us(d, m, n) < std::min(engine, cores)) return GemmRoute::kFew;
  }
  if (cores_ok && (forced || !gemm_few_tokens_by_engine(d, f, m, n, k))) return GemmRoute::kCores;
  return GemmRoute::kOther;
}

hipError_t launch_gemm_like(Fmt f, hipStream_t stream, uint64_t a, uint64_t w, uint64_t c, uint32_t m, uint32_t n,
                            uint32_t k, bool is_gemv, uint32_t flags = 0) {
  if (k % 256u != 0) return hipErrorInvalidValue;
  if (n == 0 || m == 0) return hipSuccess;
  if ((a == 0 && k != 0) || c == 0 || (w == 0 && k != 0)) return hipErrorInvalidValue;
  DeviceKernels* d = nullptr;
  hipError_t e = device_kernels(&d);
  if (e != hipSuccess) return e;
  if (!is_gemv) {
    const GemmRoute route = gemm_route(*d, f, a, w, c, m, n, k);
    if (route == GemmRoute::kFew) return launch_gemm_few(d, stream, a, w, c, m, n, k);
    if (route == GemmRoute::kCores) return launch_kq_gemm_f16(d, f, stream, a, w, c, m, n, k);
  }
  const uint32_t grid_y = std::min<uint32_t>(m, 65535u);
  // GEMV parameter order is (y, w, x, k, n); GEMM is (a, b_quant, c, m, n, k)
  void* gemv_args[] = {&c, &w, &a, &k, &n, &flags};   // the by-name kernel takes the first five
  void* gemm_args[] = {&a, &w, &c, &m, &n, &k};
  void** args = is_gemv ? gemv_args : gemm_args;
  // A large matrix alone is 2-5 us faster as a launch of the list kernel with one entry (workgroups of 8 waves that hand
  // their rows out among themselves) than through the single kernel: Q6_K 32000 x 4096, 108 MB, 22.7 against 27.2 us.
  if (is_gemv && flags == 0 && !g_tune_group_off && double(n) * (k / 256u) * kSbBytes[f] >= kBigAloneBytes) {
    trn_gemv_desc one{};
    one.fmt = uint32_t(f) + 4u; one.k = k; one.n = n; one.y = c; one.w = w; one.x = a;
    if (list_groupable(d, one)) return launch_gemv_group(d, stream, &one, 1);
  }
  GemvGeometry g;
  if (is_gemv && gemv_fast_ok(f, c, w, a) && stream_ok(uint32_t(f) + 4u, k, n)) {
    g = stream_geometry(*d, f, k, n);
    if (g.fits) {
      flags |= kChainStreamFlag;
      return hipModuleLaunchKernel(d->gemv_flags[f], g.grid, 1u, 1, g.block, 1, 1, g.lds, stream, args, nullptr);
    }
  }
  if (k != 0 && gemv_fast_ok(f, c, w, a) && (is_gemv || (aligned(uint64_t(k) * 4u, 16) && aligned(uint64_t(n) * 4u, 4))))
    g = gemv_geometry(*d, k, n, is_gemv ? kGemvMaxWaves : 8u);   // the GEMM kernels are built for 8 waves
  if (g.fits) {
    hipFunction_t fn = is_gemv ? (flags ? d->gemv_flags[f] : d->gemv_fast[f]) : d->gemm_fast[f];
    return hipModuleLaunchKernel(fn, g.grid, is_gemv ? 1u : grid_y, 1, g.block, 1, 1, g.lds, stream, args, nullptr);
  }
  hipFunction_t fn = is_gemv ? d->gemv_generic[f] : d->gemm_generic[f];
  const uint32_t block = 256, rows_per_block = block / 64;
  const uint32_t grid = std::min<uint32_t>((n + rows_per_block - 1) / rows_per_block, uint32_t(d->cu_count) * 32u);
  return hipModuleLaunchKernel(fn, grid, is_gemv ? 1u : grid_y, 1, block, 1, 1, 0, stream, args, nullptr);
}

// The product with the GEMM family's decode as written (policy 1 of the dequantise surface): the value-by-value kernel.
hipError_t launch_gemm_as_written(Fmt f, hipStream_t stream, uint64_t a, uint64_t w, uint64_t c, uint32_t m, uint32_t n, uint32_t k) {
  if (k % 256u != 0) return hipErrorInvalidValue;
  if (n == 0 || m == 0) return hipSuccess;
  if ((a == 0 && k != 0) || c == 0 || (w == 0 && k != 0) || !aligned(a, 4) || !aligned(c, 4)) return hipErrorInvalidValue;
  DeviceKernels* d = nullptr;
  hipError_t e = device_kernels(&d);
  if (e != hipSuccess) return e;
  const uint32_t block = 256, rows_per_block = block / 64;
  const uint32_t grid = std::min<uint32_t>((n + rows_per_block - 1) / rows_per_block, uint32_t(d->cu_count) * 32u);
  void* args[] = {&a, &w, &c, &m, &n, &k};
  return hipModuleLaunchKernel(d->gemm_as_written[f], grid, std::min<uint32_t>(m, 65535u), 1, block, 1, 1, 0, stream, args, nullptr);
}

// q4k_gemm_fused: the legacy 18-byte block format (quantize.rs:151-336)
hipError_t launch_gemm_simplified(hipStream_t stream, uint64_t a, uint64_t w, uint64_t c, uint32_t m, uint32_t n, uint32_t k) {
  if (k % 32u != 0) return hipErrorInvalidValue;
  if (n == 0 || m == 0) return hipSuccess;
  if ((a == 0 && k != 0) || c == 0 || (w == 0 && k != 0) || !aligned(a, 4) || !aligned(c, 4)) return hipErrorInvalidValue;
  DeviceKernels* d = nullptr;
  hipError_t e = device_kernels(&d);
  if (e != hipSuccess) return e;
  const uint32_t block = 256, rows_per_block = block / 64;
  const uint32_t grid = std::min<uint32_t>((n + rows_per_block - 1) / rows_per_block, uint32_t(d->cu_count) * 32u);
  void* args[] = {&a, &w, &c, &m, &n, &k};
  return hipModuleLaunchKernel(d->gemm_simplified, grid, std::min<uint32_t>(m, 65535u), 1, block, 1, 1, 0, stream, args, nullptr);
}

hipError_t launch_dequant_simplified(hipStream_t stream, uint64_t out, uint64_t w, uint64_t n_blocks) {
  if (n_blocks == 0) return hipSuccess;
  if (out == 0 || w == 0 || !aligned(out, 4)) return hipErrorInvalidValue;
  DeviceKernels* d = nullptr;
  hipError_t e = device_kernels(&d);
  if (e != hipSuccess) return e;
  const uint32_t grid = uint32_t(std::min<uint64_t>((n_blocks * 32 + 255) / 256, uint64_t(d->cu_count) * 64u));
  void* args[] = {&out, &w, &n_blocks};
  return hipModuleLaunchKernel(d->dequant_simplified, grid, 1, 1, 256, 1, 1, 0, stream, args, nullptr);
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

// ---- the persistent executor behind trn_kquant_gemv_batch ---------------------------------------
struct ChainEntryHost {  // ChainEntry of kquant_chain.hip.h
  uint32_t fmt, k, n, flags;
  uint64_t w, x, y, gamma, x2, residual;
  float eps;
  uint32_t pad;
};
static_assert(sizeof(ChainEntryHost) == 72, "ChainEntry layout");
ChainEntryHost entry_of(const trn_gemv_desc& d, uint32_t extra_flags = 0u) {
  return {d.fmt, d.k, d.n, d.flags | extra_flags, d.w, d.x, d.y, d.gamma, d.x2, d.residual, d.norm_eps, 0u};
}
// an entry that folds element-wise steps in (only the quarter-block engine knows how)
bool desc_extended(const trn_gemv_desc& d) { return d.gamma || d.x2 || d.residual || (d.flags & TRN_GEMV_SWIGLU_INPUT); }
// does g read or write what p writes, or write what p reads?
bool desc_conflict(const trn_gemv_desc& g, const trn_gemv_desc& p) {
  const uint64_t reads_g[4][2] = {{g.x, 4ull * g.k}, {g.x2, g.x2 ? 4ull * g.k : 0}, {g.gamma, g.gamma ? 4ull * g.k : 0},
                                  {g.residual, g.residual ? 4ull * g.n : 0}};
  const uint64_t reads_p[4][2] = {{p.x, 4ull * p.k}, {p.x2, p.x2 ? 4ull * p.k : 0}, {p.gamma, p.gamma ? 4ull * p.k : 0},
                                  {p.residual, p.residual ? 4ull * p.n : 0}};
  auto overlap = [](uint64_t a, uint64_t alen, uint64_t b, uint64_t blen) { return alen && blen && a < b + blen && b < a + alen; };
  if (overlap(g.y, 4ull * g.n, p.y, 4ull * p.n)) return true;
  for (int i = 0; i < 4; ++i)
    if (overlap(reads_g[i][0], reads_g[i][1], p.y, 4ull * p.n) || overlap(g.y, 4ull * g.n, reads_p[i][0], reads_p[i][1])) return true;
  return false;
}

struct ChainWorkspace {
  void* d_entries = nullptr;
  size_t cap_entries = 0;
  uint32_t* d_counters = nullptr;
  size_t cap_counters = 0;
  uint32_t* h_status = nullptr;  // pinned, device-visible: set by the kernel if a barrier wait gave up
  uint32_t* d_status = nullptr;
  std::vector<ChainEntryHost> last;
  uint32_t grid = 0, block = 0, lds = 0, barriers = 0;
  // phase executor: per phase and workgroup, what to do (PhaseAssign of kquant_chain.hip.h)
  void* d_assign = nullptr;
  size_t cap_assign = 0;
  std::vector<uint32_t> last_assign;
};
std::map<std::pair<int, hipStream_t>, ChainWorkspace> g_chain_ws;

// words one barrier owns: top counter + one counter per group of 32 workgroups, 256 bytes apart
// (chain_barrier_stride of kquant_chain.hip.h)
uint32_t chain_barrier_stride_host(uint32_t num_workgroups) { return 64u * (1u + (num_workgroups + 31u) / 32u); }



// batch_mode 1: the list as phases of independent entries in ONE resident launch (kq_gemv_phases): one workgroup
// of 12 waves per CU, per phase dealt to the phase's entries in proportion to their bytes, a device-wide
// barrier between phases.  *handled = false (and hipSuccess): not possible here, issue the list the plain way.
constexpr uint32_t kGroupMax = 16;     // entries one grouped launch can hold (kGroupEntries of the kernel)
// what a further slab of 4096 columns adds to the cost of an entry's bytes when workgroups are shared out (launch_gemv_group)
constexpr double kSlabCost = 0.4;
// what a streamed entry's bytes cost against an entry's on the register path (launch_gemv_group)
constexpr double kStreamCost = 0.95;
// rows a wave must get for an entry of a launch of up to sixteen to stream: the strict decoder chain 1370 / 1381 / 1356 / 1338 / 1336 /
// 1334 us with 1 / 4 / 8 / 12 / 16 / 24 (its launches of one to three entries leave a wave 6-11 rows).  Since the register form
// asks for a wave's next row while it computes this one, the pass with shared buffers (65 launches) takes 1030 / 999 / 998 /
// 999 us with 16 / 24 / 48 / never; the strict chain does not care (1270 us).
constexpr double kGroupStreamMinRows = 24.0;
// launches of more than sixteen entries (plan_gemv_many): weight per further slab and what a piece of work costs a workgroup
// (KB of weights).  The 7B pass: 730 / 718 / 704 / 702 / 702 / 708 / 711 us with 40 / 30 / 25 / 20 / 15 / 10 / 5 % per slab (with 40 %
// the workgroups with the one-slab o matrices ended 35 us after those with the three-slab down matrices); the cost of a piece
// made no difference between 1 and 128 KB, more was slower.  With the register form's rows double-buffered and its loads
// global (the three-slab rows 8 % faster): 672 / 664 / 661 / 659 / 660 / 678 / 688 us with 18 / 16 / 14 / 13 / 10 / 22 / 26 %.
constexpr double kManySlabCost = 0.13, kManyItemKb = 64.0;
// Entries a launch takes by default: as many as the kernel holds, looked for among the next 32 of the list.  On the 7B
// pass with activation buffers per layer: 8 entries (138 MB a launch, 30 launches) 879 us, 12 of the next 24 (21
// launches) 820 us, 14 of 28 (18) 821 us, 16 of 32 (16 launches of 270 MB) 823 us; the launches of 12-16 entries run at
// 4.8-5.4 TB/s against 4.3-4.7 for 8.  (Before the workgroups of a launch were kept within the number resident at once -
// launch_gemv_group - sixteen entries measured 1075 us: shares rounded up to 260 workgroups for 256 places.)
constexpr uint32_t kGroupDefault = 16;
// Beyond kGroupMax entries a launch takes its entries from tables in device memory (launch_gemv_many): as many mutually
// independent entries as the list offers, looked for over the whole list.  The 7B pass with activation buffers per layer
// is then three launches - the 160 q, k, v, gate and up matrices (2.5 GB), the 64 o and down matrices (1.5 GB), the head -
// where sixteen entries a launch made 16 launches of 258 MB, each paying 5-7 us of fixed time over a bare read.
constexpr uint32_t kManyMax = 4096;
bool list_groupable(DeviceKernels* dk, const trn_gemv_desc& d) {
  return d.n != 0 && d.k != 0 && d.x && d.w && d.y && gemv_fast_ok(Fmt(d.fmt - 4), d.y, d.w, d.x) &&
         gemv_geometry(*dk, d.k, d.n).fits;
}

// Cuts a list into launches (mode 0).  A launch is filled with up to group_max entries that are independent of one
// another AND of every earlier entry that has not been launched yet: the first entry still waiting always goes in,
// later ones of a window are brought forward when nothing they read or write is touched by an entry they would
// overtake.  What an entry computes does not depend on the company it is launched in, so the results are those of
// the list in order.  many_ok: launches of more than kGroupMax entries may be made (not while the stream is being
// captured into a graph: their tables are uploaded by a copy).
void schedule_list(DeviceKernels* dk, const trn_gemv_desc* descs, uint32_t count, std::vector<std::vector<uint32_t>>* launches,
                   bool many_ok = true) {
  const uint32_t cap = many_ok ? kManyMax : kGroupMax;
  const uint32_t group_max = g_tune_group_off ? 1u : (g_tune_group_max > 0 ? std::min<uint32_t>(uint32_t(g_tune_group_max), cap) : cap);
  const uint32_t window = g_tune_group_off ? 1u : (g_tune_group_window > 0 ? uint32_t(g_tune_group_window) : std::max(2u * kGroupDefault, 2u * group_max));
  std::vector<uint8_t> launched(count, 0), groupable(count, 0);
  for (uint32_t i = 0; i < count; ++i) groupable[i] = list_groupable(dk, descs[i]) ? 1 : 0;
  // conflicts between an entry and the (at most window - 1) entries before it, looked up many times below
  const uint32_t span = std::min(window, count);
  std::vector<uint8_t> conf(size_t(count) * span, 0);      // conf[j * span + (j - i)] for 0 < j - i < span
  for (uint32_t j = 0; j < count; ++j)
    for (uint32_t i = j > span - 1 ? j - (span - 1) : 0; i < j; ++i)
      conf[size_t(j) * span + (j - i)] = (desc_conflict(descs[j], descs[i]) || desc_conflict(descs[i], descs[j])) ? 1 : 0;
  for (uint32_t pos = 0; pos < count;) {
    if (launched[pos]) { ++pos; continue; }
    std::vector<uint32_t> members(1, pos);
    if (groupable[pos]) {
      const uint32_t end = uint32_t(std::min<uint64_t>(count, uint64_t(pos) + window));
      for (uint32_t j = pos + 1; j < end && members.size() < group_max; ++j) {
        if (launched[j]) continue;
        if (!groupable[j]) break;                    // an entry that takes another path keeps its place in the order
        bool ok = true;
        for (uint32_t i = pos; i < j && ok; ++i)     // the members of the launch and everything it would overtake
          if (!launched[i]) ok = !conf[size_t(j) * span + (j - i)];
        if (ok) members.push_back(j);
      }
    }
    for (uint32_t m : members) launched[m] = 1;
    launches->push_back(std::move(members));
  }
}

hipError_t launch_phases(DeviceKernels* d, ChainWorkspace* ws, hipStream_t stream, const trn_gemv_desc* list,
                         uint32_t count, bool* handled) {
  constexpr uint32_t kWaves = kGemvMaxWaves;
  const uint32_t G = uint32_t(d->cu_count);
  // phases: the launches the list would be cut into (entries that are independent of one another and of what they
  // overtake), one after the other
  std::vector<std::vector<uint32_t>> cut;
  schedule_list(d, list, count, &cut);
  std::vector<trn_gemv_desc> ordered;
  std::vector<std::pair<uint32_t, uint32_t>> ph;
  for (const std::vector<uint32_t>& members : cut) {
    ph.emplace_back(uint32_t(ordered.size()), uint32_t(ordered.size() + members.size()));
    for (uint32_t mbr : members) ordered.push_back(list[mbr]);
  }
  const trn_gemv_desc* descs = ordered.data();
  const uint32_t phases = uint32_t(ph.size());
  std::vector<uint32_t> assign(size_t(phases) * G * 4u, 0u);   // entry, block_id, num_blocks, fmt
  std::vector<ChainEntryHost> entries(count);
  for (uint32_t i = 0; i < count; ++i) entries[i] = entry_of(descs[i]);
  uint32_t lds = 0;
  for (uint32_t p = 0; p < phases; ++p) {
    const uint32_t a = ph[p].first, b = ph[p].second, m = b - a;
    double total = 0.0;
    std::vector<double> bytes(m);
    for (uint32_t i = 0; i < m; ++i) {
      // cost, not bytes: a Q6_K byte takes longer than a Q4_K byte (measured: the workgroups of a Q6_K entry with
      // a byte share ended 5 us after those of its Q4_K neighbours)
      const uint32_t slabs_i = std::min((descs[a + i].k / 256u + 15u) / 16u, kWaves);
      bytes[i] = double(descs[a + i].n) * (descs[a + i].k / 256u) * kSbBytes[descs[a + i].fmt - 4] * (1.0 + kSlabCost * (slabs_i - 1u));
      total += bytes[i];
    }
    // shares: at least one workgroup each, the rest in proportion to the bytes (largest remainders first)
    std::vector<uint32_t> share(m, 1u);
    uint32_t left = G - m;
    std::vector<std::pair<double, uint32_t>> frac(m);
    for (uint32_t i = 0; i < m; ++i) {
      const double want = double(G - m) * bytes[i] / total;
      const uint32_t whole = uint32_t(want);
      share[i] += whole;
      left -= whole;
      frac[i] = {want - whole, i};
    }
    std::sort(frac.begin(), frac.end(), [](const auto& x, const auto& y) { return x.first > y.first; });
    for (uint32_t i = 0; i < left; ++i) ++share[frac[i % m].second];
    uint32_t wg = 0;
    for (uint32_t i = 0; i < m; ++i) {
      const trn_gemv_desc& e = descs[a + i];
      const uint32_t nsb = e.k / 256u, slabs = (nsb + 15u) / 16u, sw = std::min(slabs, kWaves), groups = kWaves / sw;
      // 12 waves hand their row batches out among themselves: a share need not be a whole number of rounds
      const uint32_t ug = kGemvRowsPerBatch;
      (void)groups;
      uint64_t rows = (uint64_t(e.n) + share[i] - 1) / share[i];
      rows = std::max<uint64_t>(ug, (rows + ug - 1) / ug * ug);
      const uint64_t need = uint64_t(e.k) * 4u + uint64_t(sw) * rows * 4u + kLdsScratch;
      if (need > kFastLdsLimit) return hipSuccess;
      lds = std::max<uint32_t>(lds, uint32_t(need));
      const uint32_t used = uint32_t((uint64_t(e.n) + rows - 1) / rows);
      for (uint32_t bId = 0; bId < share[i]; ++bId, ++wg) {
        uint32_t* q = &assign[(size_t(p) * G + wg) * 4u];
        if (bId < used) { q[0] = a + i; q[1] = bId; q[2] = used; q[3] = e.fmt; }
      }
    }
  }
  int occ = 0;
  if (hipModuleOccupancyMaxActiveBlocksPerMultiprocessor(&occ, d->phases, int(64u * kWaves), lds) != hipSuccess || occ < 1)
    return hipSuccess;
  hipError_t err;
  const bool same = ws->last.size() == entries.size() && ws->last_assign == assign &&
                    std::memcmp(ws->last.data(), entries.data(), entries.size() * sizeof(ChainEntryHost)) == 0;
  if (!same) {
    if ((err = hipStreamSynchronize(stream)) != hipSuccess) return err;  // a list in flight may still read the device copies
    if (ws->cap_entries < entries.size()) {
      if (ws->d_entries) (void)hipFree(ws->d_entries);
      ws->d_entries = nullptr;
      ws->cap_entries = 0;
      if ((err = hipMalloc(&ws->d_entries, entries.size() * sizeof(ChainEntryHost))) != hipSuccess) return err;
      ws->cap_entries = entries.size();
    }
    if (ws->cap_assign < assign.size()) {
      if (ws->d_assign) (void)hipFree(ws->d_assign);
      ws->d_assign = nullptr;
      ws->cap_assign = 0;
      if ((err = hipMalloc(&ws->d_assign, assign.size() * sizeof(uint32_t))) != hipSuccess) return err;
      ws->cap_assign = assign.size();
    }
    if ((err = hipMemcpy(ws->d_entries, entries.data(), entries.size() * sizeof(ChainEntryHost), hipMemcpyHostToDevice)) != hipSuccess ||
        (err = hipMemcpy(ws->d_assign, assign.data(), assign.size() * sizeof(uint32_t), hipMemcpyHostToDevice)) != hipSuccess)
      return err;
    ws->last = entries;
    ws->last_assign = assign;
  }
  const size_t n_words = size_t(phases + 1u) * chain_barrier_stride_host(G);
  if (ws->cap_counters < n_words) {
    if ((err = hipStreamSynchronize(stream)) != hipSuccess) return err;
    if (ws->d_counters) (void)hipFree(ws->d_counters);
    ws->d_counters = nullptr;
    ws->cap_counters = 0;
    if ((err = hipMalloc(reinterpret_cast<void**>(&ws->d_counters), n_words * sizeof(uint32_t))) != hipSuccess) return err;
    ws->cap_counters = n_words;
  }
  uint32_t n_counters = uint32_t(n_words), zero = 0u;
  void* fill_args[] = {&ws->d_counters, &n_counters, &zero};
  const uint32_t fill_grid = std::max(1u, std::min(64u, (n_counters + 255u) / 256u));
  if ((err = hipModuleLaunchKernel(d->fill_u32, fill_grid, 1, 1, 256, 1, 1, 0, stream, fill_args, nullptr)) != hipSuccess) return err;
  uint32_t spin_limit = g_tune_chain_spin_limit > 0 ? uint32_t(g_tune_chain_spin_limit) : 4000000u;
  uint32_t np = phases;
  void* args[] = {&ws->d_entries, &ws->d_assign, &np, &ws->d_counters, &ws->d_status, &spin_limit};
  err = hipModuleLaunchCooperativeKernel(d->phases, G, 1, 1, 64u * kWaves, 1, 1, lds, stream, args);
  if (err != hipSuccess) {
    (void)hipGetLastError();
    return hipSuccess;
  }
  ws->grid = G; ws->block = 64u * kWaves; ws->lds = lds; ws->barriers = phases;
  *handled = true;
  return hipSuccess;
}

// Runs the list as one cooperative launch when every entry qualifies for the fast kernels.
// *handled = false (and hipSuccess) means the caller should issue the entries one by one.
hipError_t launch_chain(hipStream_t stream, const trn_gemv_desc* descs, uint32_t count, bool* handled) {
  *handled = false;
  if (g_tune_batch_mode == 0 || count < 2) return hipSuccess;
  DeviceKernels* d = nullptr;
  hipError_t e = device_kernels(&d);
  if (e != hipSuccess) return e;
  if (!d->cooperative) return hipSuccess;
  for (uint32_t i = 0; i < count; ++i) {
    const trn_gemv_desc& g = descs[i];
    if (g.n == 0 || g.k == 0 || !g.x || !g.w || !g.y) return hipSuccess;
    if (!gemv_fast_ok(Fmt(g.fmt - 4), g.y, g.w, g.x)) return hipSuccess;
  }
  int dev = 0;
  if ((e = hipGetDevice(&dev)) != hipSuccess) return e;
  std::lock_guard<std::mutex> lock(g_ws_mutex);   // across the workspace's growth, the uploads and the launch
  ChainWorkspace* ws = &g_chain_ws[std::make_pair(dev, stream)];
  if (!ws->h_status) {
    if ((e = hipHostMalloc(reinterpret_cast<void**>(&ws->h_status), 64, hipHostMallocMapped)) != hipSuccess) return e;
    ws->h_status[0] = 0;
    if ((e = hipHostGetDevicePointer(reinterpret_cast<void**>(&ws->d_status), ws->h_status, 0)) != hipSuccess) return e;
  }
  if (ws->h_status[0] != 0) {  // an earlier list on this stream gave up at a wait: report it once
    ws->h_status[0] = 0;
    return static_cast<hipError_t>(TRN_ERROR_WAIT_ABANDONED);
  }

  return launch_phases(d, ws, stream, descs, count, handled);
}

}  // namespace

struct trn_ctx_s {
  int device;
};
struct trn_function_s {
  hipFunction_t fn;
  int kind;
  int fmt;
  // what the reference compiles into the PTX of one kernel instance (trn_function_set_rmsnorm / _set_attention)
  bool has_constants;
  uint32_t hidden_size;
  float epsilon;
  uint32_t head_dim, num_heads, num_kv_heads, max_seq_len;
  float scale;
};
struct trn_module_s {
  hipModule_t module;
  bool builtin;
  std::mutex mutex;
  std::map<std::string, trn_function_s*> functions;
};
struct trn_event_s {
  hipEvent_t ev;
  hipStream_t stream;   // where it was recorded last
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
  name[0] = 0;
  hipError_t e = hipDeviceGetName(name, len, static_cast<hipDevice_t>(device));
  if (e != hipSuccess) return st(e);
  if (name[0] == 0) {   // some driver stacks leave the marketing name empty: fall back to the ISA name
    hipDeviceProp_t prop;
    e = hipGetDeviceProperties(&prop, static_cast<int>(device));
    if (e != hipSuccess) return st(e);
    const char* src = prop.name[0] ? prop.name : prop.gcnArchName;
    snprintf(name, static_cast<size_t>(len), "%s", src);
  }
  return TRN_SUCCESS;
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
  TRN_TRY(hipSetDevice(ctx->device));
  // first use of the device: load the kernels and find this GPU's static scratch buffer now, so that no launcher has
  // to (one of them promises to allocate nothing)
  DeviceKernels* d = nullptr;
  return st(device_kernels(&d));
}

trn_status trn_ctx_synchronize(void) {
  TRN_TRY(hipDeviceSynchronize());
  int dev = 0;
  TRN_TRY(hipGetDevice(&dev));
  trn_status waited = TRN_SUCCESS;      // every stream of the device is idle now: report (once) any abandoned wait
  std::lock_guard<std::mutex> lock(g_ws_mutex);
  for (auto& kv : g_chain_ws)
    if (kv.first.first == dev && kv.second.h_status && kv.second.h_status[0] != 0) {
      kv.second.h_status[0] = 0;
      waited = TRN_ERROR_WAIT_ABANDONED;
    }
  return waited;
}

// ---- 4. modules --------------------------------------------------------------------------
// Is `image` (an ELF code object in host memory) a copy of the built-in one?  The length comes from the image's own
// ELF header (section header table at the end), so nothing is read beyond what the loader itself would read.
static bool image_is_builtin(const void* image) {
  if (image == static_cast<const void*>(trn_builtin_hsaco_begin)) return true;
  const unsigned char* p = static_cast<const unsigned char*>(image);
  const size_t builtin_size = size_t(trn_builtin_hsaco_end - trn_builtin_hsaco_begin);
  if (builtin_size < 64 || std::memcmp(p, trn_builtin_hsaco_begin, 64) != 0) return false;   // Elf64_Ehdr, e_shoff included
  uint64_t shoff;
  uint16_t shentsize, shnum;
  std::memcpy(&shoff, p + 40, 8);
  std::memcpy(&shentsize, p + 58, 2);
  std::memcpy(&shnum, p + 60, 2);
  const uint64_t elf_size = shoff + uint64_t(shentsize) * shnum;
  return elf_size <= builtin_size && elf_size >= 64 && std::memcmp(p, trn_builtin_hsaco_begin, size_t(elf_size)) == 0;
}

trn_status trn_module_load_data(trn_module* module, const void* image) {
  if (!module || !image) return TRN_ERROR_INVALID_VALUE;
  hipModule_t m = nullptr;
  TRN_TRY(hipModuleLoadData(&m, image));
  trn_module_s* h = new trn_module_s();
  h->module = m;
  // the built-in image handed back through trn_builtin_image gets the same treatment as trn_module_load_builtin:
  // its kernels keep their own geometry however the caller launches them
  h->builtin = image_is_builtin(image);
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
  trn_function_s* h = new trn_function_s{f, KIND_OTHER, 0, false, 0u, 0.0f, 0u, 0u, 0u, 0u, 0.0f};
  if (module->builtin) {
    h->kind = KIND_INTERNAL;
    const std::string n = name;
    for (int i = 0; i < NFMT; ++i) {
      if (n == std::string(kFmtName[i]) + "_gemv_warp_reduce") { h->kind = KIND_GEMV; h->fmt = i; }
      if (n == std::string(kFmtName[i]) + "_gemm_ggml") { h->kind = KIND_GEMM; h->fmt = i; }
    }
    if (n == "q4k_gemm_fused") h->kind = KIND_GEMM_SIMPLIFIED;
    if (n == "gemv_warp_reduce" || n == "gemv_coalesced") h->kind = KIND_GEMV_F32;
    if (n == "incremental_attention") h->kind = KIND_ATTENTION;
    if (n == "residual_add") h->kind = KIND_RESIDUAL_ADD;
    if (n == "fused_swiglu") h->kind = KIND_SWIGLU;
    if (n == "rmsnorm") h->kind = KIND_RMSNORM;
    if (n == "fused_residual_rmsnorm") h->kind = KIND_RESIDUAL_RMSNORM;
  }
  module->functions[name] = h;
  *func = h;
  return TRN_SUCCESS;
}

trn_status trn_function_set_rmsnorm(trn_function func, uint32_t hidden_size, float epsilon) {
  if (!func || (func->kind != KIND_RMSNORM && func->kind != KIND_RESIDUAL_RMSNORM) || !(epsilon >= 0.0f)) return TRN_ERROR_INVALID_VALUE;
  func->hidden_size = hidden_size;
  func->epsilon = epsilon;
  func->has_constants = true;
  return TRN_SUCCESS;
}

trn_status trn_function_set_attention(trn_function func, uint32_t head_dim, uint32_t num_heads, uint32_t num_kv_heads,
                                      uint32_t max_seq_len, float scale) {
  if (!func || func->kind != KIND_ATTENTION) return TRN_ERROR_INVALID_VALUE;
  func->head_dim = head_dim;
  func->num_heads = num_heads;
  func->num_kv_heads = num_kv_heads;
  func->max_seq_len = max_seq_len;
  func->scale = scale;
  func->has_constants = true;
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

namespace {
void release_list_plans(hipStream_t stream);      // the cached plans of trn_kquant_gemv_batch and their device tables (defined with them)
}
// The per-(device, stream) scratch buffers of a stream that is going away (partial sums, arrival counters, the
// resident executor's tables).  The stream must be idle.
static void release_stream_workspaces(hipStream_t stream) {
  std::lock_guard<std::mutex> lock(g_ws_mutex);
  auto drop_simple = [&](auto& map) {
    for (auto it = map.begin(); it != map.end();) {
      if (it->first.second == stream) {
        if (it->second.buf) (void)hipFree(it->second.buf);
        it = map.erase(it);
      } else {
        ++it;
      }
    }
  };
  drop_simple(g_gemv_f32_ws);
  drop_simple(g_attention_ws);
  drop_simple(g_gemm_ws);
  release_list_plans(stream);
  for (auto it = g_chain_ws.begin(); it != g_chain_ws.end();) {
    if (it->first.second == stream) {
      ChainWorkspace& w = it->second;
      if (w.d_entries) (void)hipFree(w.d_entries);
      if (w.d_counters) (void)hipFree(w.d_counters);
      if (w.d_assign) (void)hipFree(w.d_assign);
      if (w.h_status) (void)hipHostFree(w.h_status);
      it = g_chain_ws.erase(it);
    } else {
      ++it;
    }
  }
}

// A resident executor whose device-side wait ran out of its spin budget leaves a mark in the stream's status word and
// exits; the work behind it on the stream still runs, on stale data.  Every call that tells the caller "the stream's
// work is done" looks at the word, clears it and reports TRN_ERROR_WAIT_ABANDONED once.
static trn_status take_wait_status(hipStream_t stream) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return TRN_SUCCESS;
  std::lock_guard<std::mutex> lock(g_ws_mutex);
  auto it = g_chain_ws.find(std::make_pair(dev, stream));
  if (it == g_chain_ws.end() || !it->second.h_status || it->second.h_status[0] == 0) return TRN_SUCCESS;
  it->second.h_status[0] = 0;
  return TRN_ERROR_WAIT_ABANDONED;
}

trn_status trn_stream_destroy(trn_stream stream) {
  if (!stream) return TRN_ERROR_INVALID_VALUE;
  hipStream_t s = static_cast<hipStream_t>(stream);
  // work that still uses the stream's scratch buffers must have finished before they are freed
  const hipError_t e = hipStreamSynchronize(s);
  const trn_status waited = take_wait_status(s);
  release_stream_workspaces(s);
  const hipError_t d = hipStreamDestroy(s);
  if (e != hipSuccess) return st(e);
  return d != hipSuccess ? st(d) : waited;
}

trn_status trn_stream_synchronize(trn_stream stream) {
  TRN_TRY(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
  return take_wait_status(static_cast<hipStream_t>(stream));
}

trn_status trn_launch_kernel(trn_function func, unsigned grid_x, unsigned grid_y, unsigned grid_z, unsigned block_x,
                             unsigned block_y, unsigned block_z, unsigned shared_mem_bytes, trn_stream stream,
                             void** kernel_params, void** extra) {
  if (!func) return TRN_ERROR_INVALID_VALUE;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (func->kind == KIND_GEMV || func->kind == KIND_GEMM || func->kind == KIND_GEMM_SIMPLIFIED) {
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
    if (func->kind == KIND_GEMM_SIMPLIFIED) return st(launch_gemm_simplified(s, p0, p1, p2, m, n, k));
    return st(launch_gemm_like(Fmt(func->fmt), s, p0, p1, p2, m, n, k, false));
  }
  if (func->kind == KIND_INTERNAL) return TRN_ERROR_INVALID_VALUE;   // only the typed entry points launch these
  if (func->kind == KIND_ATTENTION) {      // (q_ptr, k_ptr, v_ptr, out_ptr, seq_len): attention.rs:897-901, nothing beyond
    if (!kernel_params || !func->has_constants) return TRN_ERROR_INVALID_VALUE;
    for (int i = 0; i < 5; ++i)
      if (!kernel_params[i]) return TRN_ERROR_INVALID_VALUE;
    uint64_t p[4];
    uint32_t seq_len;
    for (int i = 0; i < 4; ++i) std::memcpy(&p[i], kernel_params[i], 8);
    std::memcpy(&seq_len, kernel_params[4], 4);
    return st(launch_attention(s, p[0], p[1], p[2], p[3], seq_len, func->head_dim, func->num_heads, func->num_kv_heads,
                               func->max_seq_len, func->scale));
  }
  if (func->kind == KIND_GEMV_F32) {                                           // (y, a, x, k_dim, n_dim)
    if (!kernel_params) return TRN_ERROR_INVALID_VALUE;
    for (int i = 0; i < 5; ++i)
      if (!kernel_params[i]) return TRN_ERROR_INVALID_VALUE;
    uint64_t p0, p1, p2;
    uint32_t k, n;
    std::memcpy(&p0, kernel_params[0], 8);
    std::memcpy(&p1, kernel_params[1], 8);
    std::memcpy(&p2, kernel_params[2], 8);
    std::memcpy(&k, kernel_params[3], 4);
    std::memcpy(&n, kernel_params[4], 4);
    return st(launch_gemv_f32(s, p0, p1, p2, k, n));
  }
  if (func->kind == KIND_RESIDUAL_ADD || func->kind == KIND_SWIGLU) {          // (ptr, ptr, output_ptr, n)
    if (!kernel_params || !kernel_params[0] || !kernel_params[1] || !kernel_params[2] || !kernel_params[3]) return TRN_ERROR_INVALID_VALUE;
    uint64_t p0, p1, p2;
    uint32_t n;
    std::memcpy(&p0, kernel_params[0], 8);
    std::memcpy(&p1, kernel_params[1], 8);
    std::memcpy(&p2, kernel_params[2], 8);
    std::memcpy(&n, kernel_params[3], 4);
    return st(launch_elementwise(Kind(func->kind), s, p0, p1, p2, n));
  }
  if (func->kind == KIND_RMSNORM || func->kind == KIND_RESIDUAL_RMSNORM) {
    // (input, output, gamma) layernorm.rs:426-428 / (residual, input, output, gamma) elementwise.rs:146-149; the row
    // length and epsilon are constants of the kernel instance (trn_function_set_rmsnorm), never read from the array
    const int np = func->kind == KIND_RMSNORM ? 3 : 4;
    if (!kernel_params || !func->has_constants) return TRN_ERROR_INVALID_VALUE;
    for (int i = 0; i < np; ++i)
      if (!kernel_params[i]) return TRN_ERROR_INVALID_VALUE;
    uint64_t p[4] = {0, 0, 0, 0};
    for (int i = 0; i < np; ++i) std::memcpy(&p[i], kernel_params[i], 8);
    if (np == 3) return st(launch_rmsnorm(s, 0, p[0], p[1], p[2], func->hidden_size, func->epsilon, false));
    return st(launch_rmsnorm(s, p[0], p[1], p[2], p[3], func->hidden_size, func->epsilon, true));
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

namespace {
struct GemvGroupHost {   // GemvGroup of kquant_kernels.hip: what a workgroup's first loads need, then the rest
  struct Hot { uint64_t w, x; uint32_t k, n, fmt, flags, first_block, num_blocks; } hot[kGroupMax];
  struct Cold { uint64_t y, gamma, x2, residual; float eps; uint32_t pad; } cold[kGroupMax];
};
static_assert(sizeof(GemvGroupHost) == kGroupMax * (40 + 40), "GemvGroup layout");

bool gemv_depends(const trn_gemv_desc& g, const trn_gemv_desc& p) { return desc_conflict(g, p); }

// Entries first .. first+len-1 of an array (len in 1..kGroupMax, mutually independent, all meeting the fast kernels'
// preconditions) as ONE launch.  The workgroups are as large as the largest entry needs (k > 4096 wants one
// wave per slab of 4096 columns), every entry gets a share of the resident workgroups in proportion to its
// bytes, and an entry's rows are cut evenly over its share.
hipError_t launch_gemv_group(DeviceKernels* d, hipStream_t stream, const trn_gemv_desc* descs, uint32_t len) {
  uint32_t waves = 1;
  double total_bytes = 0.0;
  for (uint32_t i = 0; i < len; ++i) {
    const GemvGeometry alone = gemv_geometry(*d, descs[i].k, descs[i].n);
    if (!alone.fits) return hipErrorInvalidValue;
    waves = std::max(waves, alone.block / 64u);
  }
  // At least 8 waves to a workgroup (they hand their row batches out among themselves, and a CU stages a vector once or
  // twice instead of three times): sixteen one-slab entries of 247 MB in one launch 55.4 us with 4 waves, 51.4 with 8,
  // 50.9 with 12; the 7B pass with shared activation buffers (65 launches of three or four entries) 1070 -> 1062 us,
  // with 12 waves 1076 us.
  waves = std::max(waves, g_tune_group_waves > 0 ? std::min(uint32_t(g_tune_group_waves), kGemvMaxWaves) : 8u);
  // What an entry costs a workgroup is not only its bytes: with k > 4096 every workgroup stages a larger vector and
  // the waves that share a row meet in LDS.  Measured on [Q6_K 4096x11008 + 3 x Q4_K 4096x4096]: with shares by bytes
  // the wide entry's workgroups end 5 us after the others; counting its bytes 1.6-1.8 times is best (0.4 per
  // further slab of 4096 columns; "group_slab_weight" overrides the percentage.  The 7B pass in launches of sixteen
  // entries: 932 / 875 / 832 / 800 / 794 / 803 / 880 us with 1 / 10 / 20 / 30 / 40 / 50 / 70 percent).
  // the kernels hold 3 waves per SIMD, 12 per CU
  const uint32_t per_cu = g_tune_blocks_per_cu > 0 ? uint32_t(g_tune_blocks_per_cu) : std::max(1u, 12u / waves);
  const double target = double(d->cu_count) * per_cu;
  auto plain_cost_of = [&](const trn_gemv_desc& e) {
    const uint32_t slabs = std::min((e.k / 256u + 15u) / 16u, waves);
    const double per_slab = g_tune_slab_weight > 0 ? int(g_tune_slab_weight) / 100.0 : kSlabCost;
    return double(e.n) * (e.k / 256u) * kSbBytes[e.fmt - 4] * (1.0 + per_slab * (slabs - 1u));
  };
  double plain_total = 0.0;
  for (uint32_t i = 0; i < len; ++i) plain_total += plain_cost_of(descs[i]);
  // An entry of one slab streams its rows through LDS when the rings of all waves fit beside its vector and a wave gets
  // enough rows to make the ring pay (by the entry's share of the workgroups: a ring is filled two batches ahead and
  // its start costs what a few rows cost).
  const double min_rows = g_tune_group_stream_min_rows > 0 ? double(int(g_tune_group_stream_min_rows)) : kGroupStreamMinRows;
  bool streams[kGroupMax] = {};
  for (uint32_t i = 0; i < len; ++i) {
    const trn_gemv_desc& e = descs[i];
    const double share = std::max(1.0, target * plain_cost_of(e) / std::max(plain_total, 1.0));
    streams[i] = stream_ok(e.fmt, e.k, e.n) && double(e.n) / share / waves >= min_rows &&
                 uint64_t(e.k) * 4u + kLdsScratch + waves * 2u * stream_slot_bytes(kSbBytes[e.fmt - 4]) + kGemvRowsPerBatch * 4u <= kStreamLdsLimit;
  }
  auto cost_of_i = [&](uint32_t i) {
    // a streamed entry's bytes arrive faster than those of an entry on the register path
    const double stream_cost = g_tune_stream_cost > 0 ? int(g_tune_stream_cost) / 100.0 : kStreamCost;
    return plain_cost_of(descs[i]) * (streams[i] ? stream_cost : 1.0);
  };
  for (uint32_t i = 0; i < len; ++i) total_bytes += cost_of_i(i);
  GemvGroupHost g{};
  uint32_t first[kGroupMax + 1] = {};
  uint32_t lds = 0;
  // rows per workgroup and workgroups of entry i when it is given `share` workgroups (0 rows: it does not fit the engine)
  // an entry of one slab streams its rows through LDS when the rings of all waves fit beside its vector
  auto ring_of = [&](uint32_t i) -> uint32_t { return streams[i] ? waves * 2u * stream_slot_bytes(kSbBytes[descs[i].fmt - 4]) : 0u; };
  struct Cut { uint64_t rows; uint32_t grid; };
  auto cut_of = [&](uint32_t i, uint64_t share) {
    const trn_gemv_desc& e = descs[i];
    const uint32_t nsb = e.k / 256u, slabs = (nsb + 15u) / 16u, sw = std::min(slabs, waves), groups = waves / sw;
    const uint64_t x_bytes = uint64_t(e.k) * 4u;
    const uint32_t ring = ring_of(i);
    const uint64_t limit = ring ? kStreamLdsLimit - ring : kFastLdsLimit;
    // workgroups of 8 waves or more (and every streamed entry) hand their row batches out among the waves: a share
    // need not be a whole number of rounds of all waves
    const uint32_t ug = (waves >= 8u || ring) ? kGemvRowsPerBatch : kGemvRowsPerBatch * groups;
    uint64_t rows = (uint64_t(e.n) + share - 1) / share;
    rows = std::max<uint64_t>(ug, (rows + ug - 1) / ug * ug);
    if (x_bytes + uint64_t(sw) * ug * 4u + kLdsScratch > limit) return Cut{0u, 0u};
    const uint64_t max_rows = (limit - kLdsScratch - x_bytes) / (uint64_t(sw) * 4u) / ug * ug;
    rows = std::min<uint64_t>(rows, max_rows);
    return Cut{rows, uint32_t((uint64_t(e.n) + rows - 1) / rows)};
  };
  uint64_t share[kGroupMax] = {};
  Cut cut[kGroupMax] = {};
  uint64_t total_grid = 0;
  for (uint32_t i = 0; i < len; ++i) {
    share[i] = std::max<uint64_t>(1, uint64_t(target * cost_of_i(i) / total_bytes + 0.5));
    cut[i] = cut_of(i, share[i]);
    if (cut[i].rows == 0) return hipErrorInvalidValue;
    total_grid += cut[i].grid;
  }
  // Rounded shares can add up to a few workgroups more than are resident at once, and a workgroup that has to wait for
  // a place runs when the others are done: the launch takes twice as long (measured: 66 us instead of 44 for twelve
  // entries in 260 workgroups of 12 waves on 256 CUs).  Take workgroups from the entries that have the most until
  // all fit.
  for (uint32_t guard = 0; total_grid > uint64_t(target) && guard < 4096u; ++guard) {
    uint32_t big = 0;
    for (uint32_t i = 1; i < len; ++i)
      if (cut[i].grid > cut[big].grid) big = i;
    if (cut[big].grid <= 1u || share[big] <= 1u) break;
    const uint32_t before = cut[big].grid;
    do cut[big] = cut_of(big, --share[big]); while (share[big] > 1u && cut[big].grid >= before);
    if (cut[big].grid >= before) break;            // (its rows per workgroup are at the limit of LDS)
    total_grid -= before - cut[big].grid;
  }
  // ... and where places are left over, give them to the entries whose workgroups have the most to do
  for (uint32_t guard = 0; total_grid < uint64_t(target) && guard < 4096u; ++guard) {
    int best = -1;
    double most = 0.0;
    Cut best_cut{};
    uint64_t best_share = 0;
    for (uint32_t i = 0; i < len; ++i) {
      const double per_wg = cost_of_i(i) / double(descs[i].n) * double(cut[i].rows);
      if (per_wg <= most) continue;
      uint64_t sh = share[i];
      Cut c = cut[i];
      while (c.grid <= cut[i].grid && sh < share[i] + 16u) c = cut_of(i, ++sh);       // the next share that changes the cut
      if (c.grid <= cut[i].grid || total_grid - cut[i].grid + c.grid > uint64_t(target)) continue;
      best = int(i); most = per_wg; best_cut = c; best_share = sh;
    }
    if (best < 0) break;
    total_grid += best_cut.grid - cut[best].grid;
    cut[best] = best_cut;
    share[best] = best_share;
  }
  for (uint32_t i = 0; i < len; ++i) {
    const trn_gemv_desc& e = descs[i];
    const uint32_t nsb = e.k / 256u, slabs = (nsb + 15u) / 16u, sw = std::min(slabs, waves);
    const uint32_t ring = ring_of(i);
    g.hot[i] = {e.w, e.x, e.k, e.n, e.fmt, e.flags | (ring ? kChainStreamFlag : 0u), 0u, 0u};
    g.cold[i] = {e.y, e.gamma, e.x2, e.residual, e.norm_eps, 0u};
    lds = std::max<uint32_t>(lds, uint32_t(uint64_t(e.k) * 4u + uint64_t(sw) * cut[i].rows * 4u + kLdsScratch + ring));
    first[i + 1] = first[i] + cut[i].grid;
    g.hot[i].first_block = first[i];
    g.hot[i].num_blocks = cut[i].grid;
  }
  for (uint32_t i = len; i < kGroupMax; ++i) first[i + 1] = first[len];   // entries that do not exist own no workgroup
  if (first[len] > 0xFFFFu) return hipErrorInvalidValue;                  // the table holds 16 bits per entry
  uint32_t packed[8];
  for (uint32_t a = 0; a < 8; ++a) packed[a] = first[2 * a + 1] | first[2 * a + 2] << 16;
  void* args[] = {&packed[0], &packed[1], &packed[2], &packed[3], &packed[4], &packed[5], &packed[6], &packed[7], &g};
  return hipModuleLaunchKernel(d->gemv_group, first[len], 1, 1, 64u * waves, 1, 1, lds, stream, args, nullptr);
}

// ---- launches of more than kGroupMax entries: tables in device memory (kq_gemv_many) ------------------------------
struct ManyTables {
  std::vector<uint32_t> host;     // [2 per workgroup: first item, items][4 per item: entry, row0, rows, 0][Hot per entry][Cold per entry]
  void* dev = nullptr;
  uint32_t grid = 0, block = 0, lds = 0;
  size_t off_items = 0, off_hot = 0, off_cold = 0;     // in bytes
};

// Cuts the rows of len mutually independent entries (all meeting the fast kernels' preconditions) into items for one
// workgroup per place on the chip: the entries lie one behind the other on an axis of cost (bytes, weighted as in
// launch_gemv_group), the axis is cut into equal parts, and a workgroup's items are the pieces of entries inside its
// part - whole batches of rows; a piece of fewer than 32 rows at either end of an entry goes to the neighbour, and an
// item holds no more rows than its partial sums have room for in LDS.
hipError_t plan_gemv_many(DeviceKernels* d, const trn_gemv_desc* descs, uint32_t len, ManyTables* t) {
  // twelve waves to a workgroup, one workgroup per CU (the 7B pass: 764 us with eight, 752 us with twelve; the short
  // launches of launch_gemv_group are the other way round)
  uint32_t waves = g_tune_many_waves > 0 ? std::min(uint32_t(g_tune_many_waves), kGemvMaxWaves) : kGemvMaxWaves;
  for (uint32_t i = 0; i < len; ++i) {
    const GemvGeometry alone = gemv_geometry(*d, descs[i].k, descs[i].n);
    if (!alone.fits) return hipErrorInvalidValue;
    waves = std::max(waves, alone.block / 64u);
  }
  const uint32_t G = uint32_t(d->cu_count) * (g_tune_blocks_per_cu > 0 ? uint32_t(g_tune_blocks_per_cu) : std::max(1u, 12u / waves));
  const uint32_t ug = kGemvRowsPerBatch;
  struct Ent { double cost; uint32_t ring, sw, max_rows; uint64_t x_bytes; };
  std::vector<Ent> ent(len);
  double total = 0.0;
  for (uint32_t i = 0; i < len; ++i) {
    const trn_gemv_desc& e = descs[i];
    const uint32_t slabs = (e.k / 256u + 15u) / 16u, sw = std::min(slabs, waves);
    uint32_t ring = stream_ok(e.fmt, e.k, e.n) ? waves * 2u * stream_slot_bytes(kSbBytes[e.fmt - 4]) : 0u;
    const uint64_t x_bytes = uint64_t(e.k) * 4u;
    if (ring && x_bytes + kLdsScratch + ring + ug * 4u > kStreamLdsLimit) ring = 0u;
    const uint64_t limit = ring ? kStreamLdsLimit - ring : kFastLdsLimit;
    if (x_bytes + uint64_t(sw) * ug * 4u + kLdsScratch > limit) return hipErrorInvalidValue;
    const uint32_t max_rows = uint32_t(std::min<uint64_t>((limit - kLdsScratch - x_bytes) / (uint64_t(sw) * 4u) / ug * ug, 1u << 20));
    const double per_slab = g_tune_many_slab_weight > 0 ? int(g_tune_many_slab_weight) / 100.0 : kManySlabCost;
    const double stream_cost = g_tune_stream_cost > 0 ? int(g_tune_stream_cost) / 100.0 : kStreamCost;
    const double cost = double(e.n) * (e.k / 256u) * kSbBytes[e.fmt - 4] * (1.0 + per_slab * (sw - 1u)) * (ring ? stream_cost : 1.0);
    ent[i] = {cost, ring, sw, max_rows, x_bytes};
    total += cost;
  }
  // Every piece of an entry that a workgroup takes costs it a start of its own (the vector staged, the first batches on
  // their way, the last ones summed with nothing behind them): item_cost, in the axis's bytes.  The workgroups are filled
  // one after the other up to their share of the axis so far, so that what one leaves over the next ones get.
  const double item_cost = (g_tune_many_item_kb > 0 ? double(int(g_tune_many_item_kb)) : kManyItemKb) * 1024.0;
  const double part = (total + item_cost * (double(len) + double(G))) / G;
  std::vector<std::vector<uint32_t>> items_of(G);      // per workgroup: (entry, row0, rows) triples
  uint32_t lds = 0;
  double assigned = 0.0;
  uint32_t i = 0, row = 0;
  for (uint32_t w = 0; w < G && i < len; ++w) {
    const bool last = w + 1u == G;
    while (i < len) {
      const trn_gemv_desc& e = descs[i];
      const double per_row = ent[i].cost / double(e.n);
      const uint32_t left = e.n - row;
      uint32_t take = left;
      if (!last) {
        const double budget = double(w + 1u) * part - assigned - item_cost;
        take = budget <= 0.0 ? 0u : uint32_t(std::min<double>(double(left), budget / per_row + 0.5)) / ug * ug;
        if (take < 32u && !items_of[w].empty()) break;      // too small a piece: the next workgroup takes it
        take = std::max(take, std::min(left, 32u));          // (a workgroup with nothing yet takes something)
        if (left - take < 32u) take = left;                  // a small rest at the entry's end stays with this one
      }
      for (uint32_t done = 0; done < take;) {
        const uint32_t rows = std::min((take - done + ug - 1u) / ug * ug, ent[i].max_rows);
        items_of[w].insert(items_of[w].end(), {i, row + done, rows});
        lds = std::max<uint32_t>(lds, uint32_t(ent[i].x_bytes + uint64_t(ent[i].sw) * rows * 4u + kLdsScratch + ent[i].ring));
        done += rows;
      }
      assigned += item_cost + per_row * take;
      row += take;
      if (row >= e.n) { ++i; row = 0; }
      if (!last && assigned >= double(w + 1u) * part - item_cost) break;
    }
  }
  size_t n_items = 0;
  for (const auto& v : items_of) n_items += v.size() / 3u;
  const size_t words = 2u * size_t(G) + 4u * n_items + 20u * size_t(len);
  t->host.assign(words, 0u);
  t->off_items = 8u * size_t(G);
  t->off_hot = t->off_items + 16u * n_items;
  t->off_cold = t->off_hot + 40u * size_t(len);
  uint32_t next = 0;
  for (uint32_t w = 0; w < G; ++w) {
    t->host[2u * w] = next;
    t->host[2u * w + 1u] = uint32_t(items_of[w].size() / 3u);
    for (size_t k = 0; k < items_of[w].size(); k += 3, ++next) {
      uint32_t* it = &t->host[t->off_items / 4u + 4u * next];
      it[0] = items_of[w][k]; it[1] = items_of[w][k + 1]; it[2] = items_of[w][k + 2];
    }
  }
  for (uint32_t i = 0; i < len; ++i) {
    const trn_gemv_desc& e = descs[i];
    const GemvGroupHost::Hot hot = {e.w, e.x, e.k, e.n, e.fmt, e.flags | (ent[i].ring ? kChainStreamFlag : 0u), 0u, 0u};
    const GemvGroupHost::Cold cold = {e.y, e.gamma, e.x2, e.residual, e.norm_eps, 0u};
    std::memcpy(reinterpret_cast<uint8_t*>(t->host.data()) + t->off_hot + 40u * i, &hot, 40);
    std::memcpy(reinterpret_cast<uint8_t*>(t->host.data()) + t->off_cold + 40u * i, &cold, 40);
  }
  t->grid = G;
  t->block = 64u * waves;
  t->lds = lds;
  return hipSuccess;
}

// What trn_kquant_gemv_batch does with a list, kept per (device, stream) for as long as the same list comes again (a
// decoder issues the same list for every token): the cut into launches and the device tables of the large launches.
struct PlannedLaunch {
  std::vector<uint32_t> members;
  ManyTables many;             // used when the launch has more than kGroupMax entries
};
struct ListPlan {
  std::vector<trn_gemv_desc> key;
  int epoch = -1;
  uint64_t used = 0;           // when it was used last (g_plan_clock)
  bool in_a_graph = false;     // a stream capture has recorded launches that read this plan's device tables
  std::vector<PlannedLaunch> launches;
};
// A few plans per stream (a decoder may issue the layers' lists one by one, or alternate between lists): the one used
// longest ago makes room for a new list.
constexpr size_t kPlansPerStream = 8;
uint64_t g_plan_clock = 0;
std::map<std::tuple<int, hipStream_t, bool>, std::vector<ListPlan>> g_list_plans;     // by device, stream and "may make large launches"; under g_ws_mutex

// Tables that a captured graph may still read are never freed (a graph can be replayed for as long as the process
// lives, on any stream): they are a few hundred KB per list, and there are as many as lists were captured.
size_t g_table_bytes_left_to_graphs = 0;
void free_plan_tables(ListPlan* plan) {
  for (PlannedLaunch& l : plan->launches)
    if (l.many.dev) {
      if (plan->in_a_graph) g_table_bytes_left_to_graphs += l.many.host.size() * 4u;
      else (void)hipFree(l.many.dev);
      l.many.dev = nullptr;
    }
  plan->in_a_graph = false;
}
void release_list_plans(hipStream_t stream) {       // under g_ws_mutex; the stream is idle
  for (auto it = g_list_plans.begin(); it != g_list_plans.end();) {
    if (std::get<1>(it->first) == stream) {
      for (ListPlan& p : it->second) free_plan_tables(&p);
      it = g_list_plans.erase(it);
    } else {
      ++it;
    }
  }
}
}  // namespace

trn_status trn_q4k_gemm_as_written(trn_stream s, trn_dptr a, trn_dptr b_quant, trn_dptr c, uint32_t m, uint32_t n, uint32_t k) {
  return st(launch_gemm_as_written(Q4K, static_cast<hipStream_t>(s), a, b_quant, c, m, n, k));
}
trn_status trn_q5k_gemm_as_written(trn_stream s, trn_dptr a, trn_dptr b_quant, trn_dptr c, uint32_t m, uint32_t n, uint32_t k) {
  return st(launch_gemm_as_written(Q5K, static_cast<hipStream_t>(s), a, b_quant, c, m, n, k));
}
trn_status trn_q6k_gemm_as_written(trn_stream s, trn_dptr a, trn_dptr b_quant, trn_dptr c, uint32_t m, uint32_t n, uint32_t k) {
  return st(launch_gemm_as_written(Q6K, static_cast<hipStream_t>(s), a, b_quant, c, m, n, k));
}

trn_status trn_q4k_gemm_fused(trn_stream s, trn_dptr a, trn_dptr b_quant, trn_dptr c, uint32_t m, uint32_t n, uint32_t k) {
  return st(launch_gemm_simplified(static_cast<hipStream_t>(s), a, b_quant, c, m, n, k));
}

trn_status trn_q4k_simplified_dequant_f32(trn_stream s, trn_dptr out, trn_dptr w, uint64_t n_blocks) {
  return st(launch_dequant_simplified(static_cast<hipStream_t>(s), out, w, n_blocks));
}

trn_status trn_incremental_attention(trn_stream s, trn_dptr q, trn_dptr k, trn_dptr v, trn_dptr out, uint32_t seq_len,
                                     uint32_t head_dim, uint32_t num_heads, uint32_t num_kv_heads, uint32_t max_seq_len, float scale) {
  return st(launch_attention(static_cast<hipStream_t>(s), q, k, v, out, seq_len, head_dim, num_heads, num_kv_heads, max_seq_len, scale));
}
trn_status trn_q5k_from_ggml(trn_stream s, trn_dptr dst, trn_dptr src, uint64_t n_sb) {
  if (n_sb == 0) return TRN_SUCCESS;
  if (!dst || !src) return TRN_ERROR_INVALID_VALUE;
  DeviceKernels* d = nullptr;
  TRN_TRY(device_kernels(&d));
  const uint32_t grid = uint32_t(std::min<uint64_t>((n_sb + 3u) / 4u, uint64_t(d->cu_count) * 32u));
  void* args[] = {&dst, &src, &n_sb};
  return st(hipModuleLaunchKernel(d->q5k_from_ggml, grid, 1, 1, 256, 1, 1, 0, static_cast<hipStream_t>(s), args, nullptr));
}
trn_status trn_gemv_f32(trn_stream s, trn_dptr y, trn_dptr a, trn_dptr x, uint32_t k, uint32_t n) {
  return st(launch_gemv_f32(static_cast<hipStream_t>(s), y, a, x, k, n));
}
trn_status trn_residual_add(trn_stream s, trn_dptr input1, trn_dptr input2, trn_dptr output, uint32_t n) {
  return st(launch_elementwise(KIND_RESIDUAL_ADD, static_cast<hipStream_t>(s), input1, input2, output, n));
}
trn_status trn_fused_swiglu(trn_stream s, trn_dptr gate, trn_dptr up, trn_dptr output, uint32_t n) {
  return st(launch_elementwise(KIND_SWIGLU, static_cast<hipStream_t>(s), gate, up, output, n));
}
trn_status trn_rmsnorm(trn_stream s, trn_dptr input, trn_dptr output, trn_dptr gamma, uint32_t hidden_size, float epsilon) {
  return st(launch_rmsnorm(static_cast<hipStream_t>(s), 0, input, output, gamma, hidden_size, epsilon, false));
}
trn_status trn_fused_residual_rmsnorm(trn_stream s, trn_dptr residual, trn_dptr input, trn_dptr output, trn_dptr gamma,
                                      uint32_t hidden_size, float epsilon) {
  return st(launch_rmsnorm(static_cast<hipStream_t>(s), residual, input, output, gamma, hidden_size, epsilon, true));
}


trn_status trn_kquant_gemv_plan(const trn_gemv_desc* descs, uint32_t count, uint32_t* launch_of) {
  if (count == 0) return TRN_SUCCESS;
  if (!descs || !launch_of) return TRN_ERROR_INVALID_VALUE;
  DeviceKernels* dk = nullptr;
  hipError_t e = device_kernels(&dk);
  if (e != hipSuccess) return st(e);
  std::vector<std::vector<uint32_t>> launches;
  schedule_list(dk, descs, count, &launches);
  for (size_t l = 0; l < launches.size(); ++l)
    for (uint32_t m : launches[l]) launch_of[m] = uint32_t(l);
  return TRN_SUCCESS;
}

trn_status trn_kquant_gemv_batch(trn_stream s, const trn_gemv_desc* descs, uint32_t count) {
  if (count == 0) return TRN_SUCCESS;
  if (!descs) return TRN_ERROR_INVALID_VALUE;
  for (uint32_t i = 0; i < count; ++i) {  // the whole list is validated before anything is launched
    const trn_gemv_desc& g = descs[i];
    if (g.fmt < 4 || g.fmt > 6 || (g.flags & ~(TRN_GEMV_NORM_INPUT | TRN_GEMV_SWIGLU_INPUT)) != 0 || g.k % 256u != 0 ||
        ((g.flags & TRN_GEMV_SWIGLU_INPUT) != 0) != (g.x2 != 0) || !aligned(g.gamma, 16) || !aligned(g.x2, 16) ||
        !aligned(g.residual, 4) || !(g.norm_eps >= 0.0f))
      return TRN_ERROR_INVALID_VALUE;
    if (g.n != 0 && ((g.k != 0 && (!g.x || !g.w)) || !g.y)) return TRN_ERROR_INVALID_VALUE;
  }
  DeviceKernels* dk = nullptr;
  hipError_t e = device_kernels(&dk);
  if (e != hipSuccess) return st(e);
  for (uint32_t i = 0; i < count; ++i)
    // folded element-wise steps need the fast engine (x, x2, gamma 16-byte aligned; the vector and a row block in LDS)
    if (desc_extended(descs[i]) && !list_groupable(dk, descs[i])) return TRN_ERROR_INVALID_VALUE;
  hipStream_t stream = static_cast<hipStream_t>(s);
  bool handled = false;
  e = launch_chain(stream, descs, count, &handled);
  if (handled || e != hipSuccess) return st(e);
  int dev = 0;
  if ((e = hipGetDevice(&dev)) != hipSuccess) return st(e);
  // while the stream is being captured into a graph nothing may be copied or allocated: kernel-argument launches only
  hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &capturing) != hipSuccess) {
    (void)hipGetLastError();
    capturing = hipStreamCaptureStatusNone;
  }
  bool many_ok = capturing == hipStreamCaptureStatusNone;
  std::lock_guard<std::mutex> lock(g_ws_mutex);
  auto find_in = [&](std::vector<ListPlan>& list) -> ListPlan* {
    for (ListPlan& p : list)
      if (p.epoch == g_tune_epoch && p.key.size() == count && std::memcmp(p.key.data(), descs, size_t(count) * sizeof(trn_gemv_desc)) == 0) return &p;
    return nullptr;
  };
  // A capture of a list that this stream has already issued eagerly takes that plan, tables and all: nothing is built,
  // copied or allocated, and the tables are then kept for as long as the process lives (free_plan_tables).
  if (!many_ok) {
    auto eager = g_list_plans.find(std::make_tuple(dev, stream, true));
    if (eager != g_list_plans.end()) {
      if (ListPlan* p = find_in(eager->second)) {
        p->in_a_graph = true;
        many_ok = true;
      }
    }
  }
  std::vector<ListPlan>& plans = g_list_plans[std::make_tuple(dev, stream, many_ok)];      // (a capture of anything else has plans of its own)
  ListPlan* found = find_in(plans);
  const bool same = found != nullptr;
  if (!same) {
    if (plans.size() < kPlansPerStream) {
      plans.emplace_back();
      found = &plans.back();
    } else {
      found = &plans[0];
      for (ListPlan& p : plans)
        if (p.used < found->used) found = &p;
    }
  }
  ListPlan& plan = *found;
  plan.used = ++g_plan_clock;
  if (!same) {
    bool had_tables = false;
    for (const PlannedLaunch& l : plan.launches) had_tables = had_tables || l.many.dev;
    if (had_tables) {      // (never during a capture: its plans have no tables)
      if ((e = hipStreamSynchronize(stream)) != hipSuccess) return st(e);   // a launch in flight may still read the old tables
      free_plan_tables(&plan);
    }
    plan.launches.clear();
    plan.key.assign(descs, descs + count);
    plan.epoch = g_tune_epoch;
    std::vector<std::vector<uint32_t>> cut;
    schedule_list(dk, descs, count, &cut, many_ok);
    std::vector<trn_gemv_desc> group;
    for (std::vector<uint32_t>& members : cut) {
      PlannedLaunch pl;
      pl.members = std::move(members);
      if (pl.members.size() > kGroupMax) {
        group.clear();
        for (uint32_t m : pl.members) group.push_back(descs[m]);
        if ((e = plan_gemv_many(dk, group.data(), uint32_t(group.size()), &pl.many)) != hipSuccess ||
            (e = hipMalloc(&pl.many.dev, pl.many.host.size() * 4u)) != hipSuccess ||
            (e = hipMemcpy(pl.many.dev, pl.many.host.data(), pl.many.host.size() * 4u, hipMemcpyHostToDevice)) != hipSuccess) {
          if (pl.many.dev) (void)hipFree(pl.many.dev);
          free_plan_tables(&plan);
          plan.launches.clear();
          plan.key.clear();
          return st(e);
        }
      }
      plan.launches.push_back(std::move(pl));
    }
  }
  std::vector<trn_gemv_desc> group;
  for (const PlannedLaunch& pl : plan.launches) {
    const std::vector<uint32_t>& members = pl.members;
    const trn_gemv_desc& head = descs[members[0]];
    // a large matrix alone (the 108 MB head of the 7B pass) is 2-4 us faster as a group of one: workgroups of 8 waves that
    // hand their rows out among themselves; smaller ones alone (37 MB, 9 MB) are slower that way
    const bool big_single = list_groupable(dk, head) && double(head.n) * (head.k / 256u) * kSbBytes[head.fmt - 4] >= kBigAloneBytes;
    if (pl.many.dev) {
      uint64_t wgs = reinterpret_cast<uint64_t>(pl.many.dev), items = wgs + pl.many.off_items, hot = wgs + pl.many.off_hot,
               cold = wgs + pl.many.off_cold;
      void* args[] = {&wgs, &items, &hot, &cold};
      e = hipModuleLaunchKernel(dk->gemv_many, pl.many.grid, 1, 1, pl.many.block, 1, 1, pl.many.lds, stream, args, nullptr);
    } else if (members.size() >= 2 || big_single || (desc_extended(head) && list_groupable(dk, head))) {
      group.clear();
      for (uint32_t m : members) group.push_back(descs[m]);
      e = launch_gemv_group(dk, stream, group.data(), uint32_t(group.size()));
    } else {
      e = launch_gemm_like(Fmt(head.fmt - 4), stream, head.x, head.w, head.y, 1, head.n, head.k, true, head.flags);
    }
    if (e != hipSuccess) return st(e);
  }
  return TRN_SUCCESS;
}

// The Q4_K GEMM for callers that cannot allocate.  Same dispatch as trn_q4k_gemm; the matrix-core form's partial
// results and counters live in this GPU's copy of the library's static scratch buffer.  After the first use of the
// library on the device (which loads the kernels and finds the buffer) this calls nothing that allocates or frees.
trn_status trn_q4k_gemm_noalloc(trn_stream s, trn_dptr a, trn_dptr b, trn_dptr c, uint32_t m, uint32_t n, uint32_t k) {
  if (k % 256u != 0) return TRN_ERROR_INVALID_VALUE;
  if (n == 0 || m == 0) return TRN_SUCCESS;
  if ((a == 0 && k != 0) || c == 0 || (b == 0 && k != 0)) return TRN_ERROR_INVALID_VALUE;
  hipStream_t stream = static_cast<hipStream_t>(s);
  DeviceKernels* d = nullptr;
  TRN_TRY(device_kernels(&d));
  // the same choice of kernel as trn_q4k_gemm, so the same bits: only the f16 matrix-core form needs scratch at all
  if (gemm_route(*d, Q4K, a, b, c, m, n, k) != GemmRoute::kCores) return st(launch_gemm_like(Q4K, stream, a, b, c, m, n, k, false));
  int dev = 0;
  TRN_TRY(hipGetDevice(&dev));
  size_t cap = 0;
  const uint64_t base = trn_noalloc_scratch(dev, &cap);
  if (!base) return TRN_ERROR_INVALID_VALUE;
  // the cut trn_q4k_gemm would take (so the bits are its bits): refused by name when its partial sums do not fit
  const GemmCut cut = gemm_cut(*d, Q4K, m, n, k);
  const size_t part_bytes = gemm_part_bytes(cut.kparts, (m + 15u) / 16u, cut.groups, cut.waves);
  if (kGemmCounterBytes + part_bytes > cap) return TRN_ERROR_SCRATCH_TOO_SMALL;
  return st(launch_kq_gemm_f16(d, Q4K, stream, a, b, c, m, n, k, base, cap, &cut));
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
  *event = new trn_event_s{e, nullptr};
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
  event->stream = static_cast<hipStream_t>(stream);
  return st(hipEventRecord(event->ev, static_cast<hipStream_t>(stream)));
}

trn_status trn_event_synchronize(trn_event event) {
  if (!event) return TRN_ERROR_INVALID_VALUE;
  TRN_TRY(hipEventSynchronize(event->ev));
  return take_wait_status(event->stream);
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

trn_status trn_read_u128(trn_stream stream, trn_dptr src, uint64_t bytes, trn_dptr sink) {
  if (bytes % 16u != 0 || !aligned(src, 16) || !aligned(sink, 4)) return TRN_ERROR_INVALID_VALUE;
  if (bytes == 0) return TRN_SUCCESS;
  if (!src || !sink) return TRN_ERROR_INVALID_VALUE;
  DeviceKernels* d = nullptr;
  TRN_TRY(device_kernels(&d));
  uint64_t n = bytes / 16u;
  // three workgroups of four waves per CU, like the one-slab GEMV launches it is compared with
  const uint32_t grid = uint32_t(std::min<uint64_t>((n + 255) / 256, uint64_t(d->cu_count) * 3u));
  void* args[] = {&src, &n, &sink};
  return st(hipModuleLaunchKernel(d->read_u128, grid, 1, 1, 256, 1, 1, 0, static_cast<hipStream_t>(stream), args, nullptr));
}

const char* trn_error_name(trn_status status) {
  if (status == TRN_ERROR_WAIT_ABANDONED) return "TRN_ERROR_WAIT_ABANDONED";
  if (status == TRN_ERROR_SCRATCH_TOO_SMALL) return "TRN_ERROR_SCRATCH_TOO_SMALL";
  return hipGetErrorName(static_cast<hipError_t>(status));
}
const char* trn_error_string(trn_status status) {
  if (status == TRN_ERROR_SCRATCH_TOO_SMALL) return "TRN_ERROR_SCRATCH_TOO_SMALL: the product needs more than the library's static scratch buffer";
  if (status == TRN_ERROR_WAIT_ABANDONED) return "TRN_ERROR_WAIT_ABANDONED: a device-side wait of the resident list executor gave up";
  return hipGetErrorString(static_cast<hipError_t>(status));
}

trn_status trn_device_cu_count(int* count) {
  if (!count) return TRN_ERROR_INVALID_VALUE;
  int dev = 0;
  TRN_TRY(hipGetDevice(&dev));
  return st(hipDeviceGetAttribute(count, hipDeviceAttributeMultiprocessorCount, dev));
}

trn_status trn_set_tuning(const char* key, int value) {
  if (!key || value < 0) return TRN_ERROR_INVALID_VALUE;
  std::lock_guard<std::mutex> lock(g_mutex);
  ++g_tune_epoch;
  if (!std::strcmp(key, "gemv_blocks_per_cu")) { g_tune_blocks_per_cu = value; return TRN_SUCCESS; }
  if (!std::strcmp(key, "gemv_row_groups")) { g_tune_row_groups = value; return TRN_SUCCESS; }
  if (!std::strcmp(key, "batch_mode")) {
    if (value > 1) return TRN_ERROR_INVALID_VALUE;
    g_tune_batch_mode = value;
    return TRN_SUCCESS;
  }
  if (!std::strcmp(key, "chain_spin_limit")) { g_tune_chain_spin_limit = value; return TRN_SUCCESS; }
  if (!std::strcmp(key, "group_off")) { g_tune_group_off = value; return TRN_SUCCESS; }
  if (!std::strcmp(key, "gemm_mfma_off")) { g_tune_gemm_mfma_off = value; return TRN_SUCCESS; }
  if (!std::strcmp(key, "gemm_tiles")) { g_tune_gemm_tiles = value; return TRN_SUCCESS; }
  if (!std::strcmp(key, "gemm_k_parts")) { g_tune_gemm_ksplit = value; return TRN_SUCCESS; }
  if (!std::strcmp(key, "gemm_waves")) { g_tune_gemm_waves = value; return TRN_SUCCESS; }
  if (!std::strcmp(key, "group_window")) { g_tune_group_window = value; return TRN_SUCCESS; }
  if (!std::strcmp(key, "group_max")) { g_tune_group_max = value; return TRN_SUCCESS; }
  if (!std::strcmp(key, "group_waves")) { g_tune_group_waves = value; return TRN_SUCCESS; }
  if (!std::strcmp(key, "group_slab_weight")) { g_tune_slab_weight = value; return TRN_SUCCESS; }
  if (!std::strcmp(key, "attention_per_cu")) { g_tune_attention_per_cu = value; return TRN_SUCCESS; }
  if (!std::strcmp(key, "attention_min_steps")) { g_tune_attention_min_steps = value; return TRN_SUCCESS; }
  if (!std::strcmp(key, "gemv_stream_off")) { g_tune_stream_off = value; return TRN_SUCCESS; }
  if (!std::strcmp(key, "gemv_stream_waves")) { g_tune_stream_waves = value; return TRN_SUCCESS; }
  if (!std::strcmp(key, "many_waves")) { g_tune_many_waves = value; return TRN_SUCCESS; }
  if (!std::strcmp(key, "group_stream_min_rows")) { g_tune_group_stream_min_rows = value; return TRN_SUCCESS; }
  if (!std::strcmp(key, "many_item_kb")) { g_tune_many_item_kb = value; return TRN_SUCCESS; }
  if (!std::strcmp(key, "many_slab_weight")) { g_tune_many_slab_weight = value; return TRN_SUCCESS; }
  if (!std::strcmp(key, "gemv_stream_q6k")) { g_tune_stream_q6k = value; return TRN_SUCCESS; }
  if (!std::strcmp(key, "gemv_stream_cost")) { g_tune_stream_cost = value; return TRN_SUCCESS; }
  if (!std::strcmp(key, "gemv_stream_min_rows")) { g_tune_stream_min_rows = value; return TRN_SUCCESS; }
  if (!std::strcmp(key, "gemm_few")) { g_tune_gemm_few = value; return TRN_SUCCESS; }
  return TRN_ERROR_INVALID_VALUE;
}

}  // extern "C"
