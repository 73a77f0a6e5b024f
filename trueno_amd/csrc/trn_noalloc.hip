// The scratch buffer of trn_q4k_gemm_noalloc: device memory that exists for as long as the library is loaded, so the
// entry point never has to allocate.  Compiled by hipcc (host + gfx950) because the array is a device symbol of this
// file; everything else of the library's host side is plain C++ (trn_runtime.cpp).
//
// Each GPU holds its own copy of the array at its own address.  `scratch` below is, in host code, only a stand-in for
// the symbol: the address a kernel may use is what hipGetSymbolAddress returns with that GPU current, asked for once
// per device (trn_noalloc_scratch_setup) and kept.
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace {
constexpr size_t kCounterBytes = size_t(1) << 16;                    // arrival counters at the front (kGemmCounterBytes)
constexpr size_t kScratchBytes = kCounterBytes + (size_t(16) << 20);   // + partial results of the parts of K
constexpr int kMaxDevices = 64;
void* g_scratch_ptr[kMaxDevices] = {};
}  // namespace

// No `used` attribute here: clang gives a static device variable that host code names an external symbol in the code
// object, which is how hipGetSymbolAddress finds it; marked `used` it stays a local symbol and the lookup fails.
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

// Once per device, with that device current (the caller serialises): find this GPU's copy and put the counters at
// zero.  Set-up may allocate and synchronise; the entry point that uses the buffer afterwards does neither.
extern "C" __attribute__((visibility("hidden"))) hipError_t trn_noalloc_scratch_setup(int dev) {
  if (dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
  if (g_scratch_ptr[dev]) return hipSuccess;
  void* ptr = nullptr;
  hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
  if (e != hipSuccess) return e;
  if (!ptr) return hipErrorInvalidSymbol;
  if ((e = hipMemset(ptr, 0, kCounterBytes)) != hipSuccess) return e;
  g_scratch_ptr[dev] = ptr;
  return hipSuccess;
}

// The buffer of device `dev` (0 before its set-up) and its size.  No HIP call.
extern "C" __attribute__((visibility("hidden"))) uint64_t trn_noalloc_scratch(int dev, size_t* bytes) {
  *bytes = kScratchBytes;
  return dev >= 0 && dev < kMaxDevices ? reinterpret_cast<uint64_t>(g_scratch_ptr[dev]) : 0;
}
