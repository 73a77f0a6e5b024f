// Shared device helpers for the gfx950 k-quant kernels: vector types, under-aligned loads,
// wave64 reductions and the byte-wise "one value" decoders.
//
// Block layouts and decode arithmetic follow trueno-gpu/src/kernels/quantize.rs:
//   Q4_K (144 B)  d f16 @0, dmin f16 @2, sc[12] @4, qs[128] @16              (:5-14, :1237-1483)
//   Q5_K (176 B)  d @0, dmin @2, sc[12] @4, qs[128] @16, qh[32] @144          (:44-47, :1589-1693)
//   Q6_K (210 B)  ql[128] @0, qh[64] @128, sc[16] int8 @192, d f16 @208       (:1754-1769, :1806-1934)
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef uint32_t u32;
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 h16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ h16x2 as_h16x2(u32 bits) { return __builtin_bit_cast(h16x2, bits); }

enum : int { FMT_Q4K = 4, FMT_Q5K = 5, FMT_Q6K = 6 };
enum : int { POLICY_GEMV = 0, POLICY_GEMM_LEGACY = 1 };

template <int FMT> struct sb_bytes;
template <> struct sb_bytes<FMT_Q4K> { static constexpr u32 value = 144; };
template <> struct sb_bytes<FMT_Q5K> { static constexpr u32 value = 176; };
template <> struct sb_bytes<FMT_Q6K> { static constexpr u32 value = 210; };

// Loads at less than natural alignment.  gfx950 under HSA runs global memory in unaligned
// access mode, so each of these is still one global_load_dword{,x2,x4}.
struct __attribute__((packed, aligned(2))) ld128_a2 { u32x4 v; };
struct __attribute__((packed, aligned(2))) ld64_a2 { u32x2 v; };
struct __attribute__((packed, aligned(1))) ld32_a1 { u32 v; };
struct __attribute__((packed, aligned(2))) ld16_a2 { uint16_t v; };

// Every pointer these take is a weight matrix in device memory; saying so (address space 1) makes them global_load
// instructions also where the pointer came out of a table in memory and the compiler could not tell.  A generic pointer
// is a flat_load, which counts as an LDS access as well: nothing behind it can be waited for on its own, so a wave
// would wait for both of its rows before it computes the first, and for its rows before it stages the vector.  The
// engines say the same of the vectors they read and write (KQ_GLOBAL, KQ_GLOBAL_MUT).
#define KQ_GLOBAL(T, p) (reinterpret_cast<const __attribute__((address_space(1))) T*>(reinterpret_cast<uintptr_t>(p)))
#define KQ_GLOBAL_MUT(T, p) (reinterpret_cast<__attribute__((address_space(1))) T*>(reinterpret_cast<uintptr_t>(p)))
__device__ __forceinline__ u32x4 load128_a2(const uint8_t* p) { return KQ_GLOBAL(ld128_a2, p)->v; }
__device__ __forceinline__ u32x2 load64_a2(const uint8_t* p) { return KQ_GLOBAL(ld64_a2, p)->v; }
__device__ __forceinline__ u32 load32_a1(const uint8_t* p) { return KQ_GLOBAL(ld32_a1, p)->v; }
__device__ __forceinline__ u32 load16_a2(const uint8_t* p) { return KQ_GLOBAL(ld16_a2, p)->v; }
__device__ __forceinline__ u32x4 load128(const uint8_t* p) { return *KQ_GLOBAL(u32x4, p); }
__device__ __forceinline__ u32x2 load64(const uint8_t* p) { return *KQ_GLOBAL(u32x2, p); }
__device__ __forceinline__ u32 load32(const uint8_t* p) { return *KQ_GLOBAL(u32, p); }

// f16 bits -> f32, exact, subnormals kept (the reference converts with cvt.f32.f16, no .ftz:
// trueno-gpu/src/ptx/builder.rs:1241-1250).
__device__ __forceinline__ float half_bits_to_f32(u32 bits) {
  const uint16_t b16 = static_cast<uint16_t>(bits & 0xFFFFu);
  _Float16 h;
  __builtin_memcpy(&h, &b16, 2);
  return static_cast<float>(h);
}

// Hides how a word was produced, so a byte-lane mask computed once per word is not re-derived
// as one bit-field extract per value and the conversions stay v_cvt_f32_ubyte0..3.
__device__ __forceinline__ u32 opaque(u32 v) {
  asm("" : "+v"(v));
  return v;
}

__device__ __forceinline__ float ubyte0(u32 v) { return static_cast<float>(v & 0xFFu); }
__device__ __forceinline__ float ubyte1(u32 v) { return static_cast<float>((v >> 8) & 0xFFu); }
__device__ __forceinline__ float ubyte2(u32 v) { return static_cast<float>((v >> 16) & 0xFFu); }
__device__ __forceinline__ float ubyte3(u32 v) { return static_cast<float>(v >> 24); }

// ---- wave64 sum, result in every lane ------------------------------------------------
template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}

__device__ __forceinline__ float wave_sum(float v) {
  v += dpp_f32<0xB1>(v);   // quad_perm [1,0,3,2]
  v += dpp_f32<0x4E>(v);   // quad_perm [2,3,0,1]
  v += dpp_f32<0x141>(v);  // row_half_mirror
  v += dpp_f32<0x140>(v);  // row_mirror: every lane of a 16-lane row now holds the row sum
  float r0 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0));
  float r1 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 16));
  float r2 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32));
  float r3 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 48));
  return (r0 + r1) + (r2 + r3);
}

// The same sum, in the same order - ((r3 + r2) + (r1 + r0)) of the four row sums, i.e. wave_sum's bits - but valid in
// lane 63 only: the rows meet through two broadcasts of a row's last lane into the rows behind it instead of four
// reads of a lane into scalar registers and three more additions.
__device__ __forceinline__ float wave_sum_lane63(float v) {
  v += dpp_f32<0xB1>(v);
  v += dpp_f32<0x4E>(v);
  v += dpp_f32<0x141>(v);
  v += dpp_f32<0x140>(v);
  // row_bcast:15 into rows 1 and 3, row_bcast:31 into rows 2 and 3 (lanes not written keep their value)
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x142, 0xA, 0xF, false));
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x143, 0xC, 0xF, false));
  return v;
}

// ---- byte-wise decoders: one value of one super-block -----------------------------------
// Used by the generic (any alignment, any K) kernels and by the GEMM-family decode policy.
// __fmul_rn/__fsub_rn keep every PTX instruction of the reference a separate rounding.
__device__ __forceinline__ void scale_min_12bit(const uint8_t* sc, u32 j, u32& s, u32& m) {
  u32 bit = 12u * j, b = bit >> 3, sh = bit & 7u;                      // quantize.rs:1607-1635
  u32 t = (static_cast<u32>(sc[b]) | (static_cast<u32>(sc[b + 1]) << 8)) >> sh;
  s = t & 63u;
  m = (t >> 6) & 63u;
}

__device__ __forceinline__ void scale_min_k4(const uint8_t* sc, u32 j, u32& s, u32& m) {
  if (j < 4) {                                                         // quantize.rs:1306-1385
    s = sc[j] & 63u;
    m = sc[j + 4] & 63u;
  } else {
    s = (sc[j + 4] & 0xFu) | ((static_cast<u32>(sc[j - 4]) >> 6) << 4);
    m = (static_cast<u32>(sc[j + 4]) >> 4) | ((static_cast<u32>(sc[j]) >> 6) << 4);
  }
}

template <int FMT, int POLICY>
__device__ __forceinline__ float decode_value(const uint8_t* b, u32 i) {
  if constexpr (FMT == FMT_Q4K || FMT == FMT_Q5K) {
    const float d = half_bits_to_f32(static_cast<u32>(b[0]) | (static_cast<u32>(b[1]) << 8));
    const float dmin = half_bits_to_f32(static_cast<u32>(b[2]) | (static_cast<u32>(b[3]) << 8));
    const uint8_t* sc = b + 4;
    const uint8_t* qs = b + 16;
    const u32 j = i >> 5;
    u32 s, m, q;
    if constexpr (POLICY == POLICY_GEMV) {
      if constexpr (FMT == FMT_Q4K) scale_min_k4(sc, j, s, m); else scale_min_12bit(sc, j, s, m);
      const u32 in_chunk = i & 63u;                                    // quantize.rs:1443-1466
      q = (static_cast<u32>(qs[(i >> 6) * 32u + (in_chunk & 31u)]) >> (4u * (in_chunk >> 5))) & 0xFu;
      if constexpr (FMT == FMT_Q5K) q += 16u * ((static_cast<u32>(b[144 + (i >> 3)]) >> (i & 7u)) & 1u);
      const float ds = __fmul_rn(d, static_cast<float>(s));
      const float dm = __fmul_rn(dmin, static_cast<float>(m));
      return __fsub_rn(__fmul_rn(ds, static_cast<float>(q)), dm);     // :1468-1471, :1677-1682
    } else {
      scale_min_12bit(sc, j, s, m);                                    // :445-475, :727-750
      const float inv63 = 1.0f / 63.0f;                                // :480
      const float sn = __fmul_rn(static_cast<float>(s), inv63);
      const float mn = __fmul_rn(static_cast<float>(m), inv63);
      q = (static_cast<u32>(qs[i >> 1]) >> (4u * (i & 1u))) & 0xFu;    // :488-507
      if constexpr (FMT == FMT_Q5K) q += 16u * ((static_cast<u32>(b[144 + (i >> 3)]) >> (i & 7u)) & 1u);
      const float dsc = __fmul_rn(d, sn);
      const float dmm = __fmul_rn(dmin, mn);
      return __fsub_rn(__fmul_rn(dsc, static_cast<float>(q)), dmm);   // :509-514
    }
  } else {
    const float d = half_bits_to_f32(static_cast<u32>(b[208]) | (static_cast<u32>(b[209]) << 8));
    if constexpr (POLICY == POLICY_GEMV) {                             // :1829-1923
      const u32 h = i >> 7, p = i & 127u, g = p >> 5, l = p & 31u, is = l >> 4;
      const float scale = static_cast<float>(static_cast<int8_t>(b[192 + 8u * h + is + 2u * g]));
      const u32 nib = (static_cast<u32>(b[64u * h + l + 32u * (g & 1u)]) >> (4u * (g >> 1))) & 0xFu;
      const u32 q2 = (static_cast<u32>(b[128 + 32u * h + l]) >> (2u * g)) & 3u;
      const float qf = static_cast<float>(static_cast<int>(nib | (q2 << 4)) - 32);
      return __fmul_rn(__fmul_rn(d, scale), qf);
    } else {                                                           // :1009-1064
      const float scale = static_cast<float>(b[192 + (i >> 4)]);
      const u32 ql = (static_cast<u32>(b[i >> 1]) >> (4u * (i & 1u))) & 0xFu;
      const u32 q2 = (static_cast<u32>(b[128 + (i >> 2)]) >> (2u * (i & 3u))) & 3u;
      const float qf = __fsub_rn(static_cast<float>(ql + 4u * q2), 32.0f);
      return __fmul_rn(__fmul_rn(d, scale), qf);
    }
  }
}
