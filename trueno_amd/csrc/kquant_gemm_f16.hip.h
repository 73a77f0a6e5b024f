// Batched Q4_K / Q5_K GEMM on the matrix cores (gfx950, v_mfma_f32_32x32x16_f16).
//
//   C[m x n] = A[m x k] . dequant(W[n x k])^T,  c[row*n + col]      (trueno-gpu/src/kernels/quantize.rs:568-574,
//   decode of the weights as in the GEMV family, quantize.rs:1237-1483 Q4_K, :1589-1693 Q5_K)
//
// Q5_K (the reference's layout: nibbles as Q4_K, eight contiguous 12-bit (scale, min) fields, fifth bit of value i in
// bit i%8 of qh[i/8] at byte 144) runs through the same kernel: q <= 31 and s_j <= 63 keep q * s_j below 2048, still
// exact in f16; the fifth bits are joined into the nibbles' 16-bit lanes before the packed multiply (a 5-bit quant in
// the low bits of a 16-bit lane is still the subnormal q * 2^-24); rows of 176 bytes are 11 sixteen-byte pieces, an odd
// stride like Q4_K's 9, so the transposed reads stay conflict-free.
//
// f16 operands without giving up f32 accuracy:
//   * the weight operand is  q * s_j * 2^-14  (nibble q <= 15, 6-bit sub-block scale s_j <= 63): an integer
//     below 1024 times a power of two, exact in f16.  It costs one AND and one packed multiply per two weights:
//     a nibble left in place in a 16-bit lane is the f16 subnormal q * 2^-24 (bits 4..7: q * 2^-20), and the
//     packed multiply by s_j * 2^10 (s_j * 2^6) turns it into the normal number wanted;
//   * every (token, super-block) run of 256 activations is scaled by a power of two so that its largest
//     element lies in [2^14, 2^15) and each element is split in two f16 pieces, hi = f16(a),
//     lo = f16((a - hi) * 2^11): 22 bits and a sign per element, products exact in the matrix cores' f32
//     accumulators.  The pieces are two rows of the token operand, so a tile of 32 operand rows is 16 tokens.
//     The workgroup does this itself, one super-block ahead of the products, straight into LDS;
//   * the accumulators run over a whole super-block (the sub-block scales are inside the operand), then
//     tot += d * 2^E(token, super-block) * acc per (row, token, super-block);
//   * the min term  dmin * sum_j m_j * (sum of a over sub-block j)  is one more small product per super-block
//     (v_mfma_f32_32x32x8_f16: m_j against the sub-block sums, split in two pieces like a).
//
// Operand roles: A operand = token pieces (row 2*token + piece), B operand = 32 rows of W.  Lane l supplies
// A[row l%32][8 k-slots of group l/32] and B[the same k-slots][col l%32]; D[row 8*(v/4) + 4*(l/32) + v%4][col l%32]
// arrives in lane l, register v.  Which k a slot stands for is this file's choice (both operands use the same
// table): lane group g = l/32 of W row r takes the 64 bytes qs[64g .. 64g+63] of a super-block, i.e. its
// sub-blocks 4g .. 4g+3; product q = 2u + h (u = 0..7, h = 0 low / 1 high nibbles) takes bytes 8u .. 8u+7 of
// those 64 in the order 0,2,1,3,4,6,5,7 (what the two ANDs per dword leave in the 16-bit lanes).
//
// Data movement: a workgroup of 4 or 8 waves takes as many strips of 32 rows of W and a run of super-blocks.
// Per super-block it needs the 16.5 KB of token operands (shared by its waves, converted from 16 KB of A) and
// one 4.5 KB weight tile per wave, read from HBM in row-contiguous 144-byte runs straight into LDS
// (global_load_lds_dwordx4) two super-blocks ahead of the arithmetic: a wave's weight tile is copied to
// registers first and its LDS space is then the target of the tile after the next; the token operands
// alternate between two LDS stages.  The weight tile lies in LDS row by row at a stride of 9 sixteen-byte pieces, which makes the
// transposed reads (lane = row) conflict-free.  Two or three workgroups share a CU, so one workgroup's loads
// overlap the others' arithmetic.  LDS is accessed through inline asm so that the compiler does not wait for
// the loads in flight.
#pragma once
#include "kquant_common.hip.h"
#include <type_traits>

typedef _Float16 h16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 h16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

namespace gemm_f16 {

constexpr u32 kTokensPerTile = 16;
constexpr u32 kMaxWaves = 8;                   // strips of 32 rows per workgroup: 4 or 8
constexpr u32 kXpMainBytes = 16 * 1024;        // 16 products x 64 lanes x 16 bytes
constexpr u32 kXpSumBytes = 512;               // 64 lanes x 4 f16
constexpr u32 kXpFactorBytes = 64;             // 16 tokens x f32
constexpr u32 kXpStageBytes = kXpMainBytes + kXpSumBytes + kXpFactorBytes;
// weight tile of one super-block of 32 rows: SB bytes a row, PIECES sixteen-byte pieces a row, copied by DMA instructions
// of 64 pieces each (the last one half full for both formats: 288 = 4.5 x 64, 352 = 5.5 x 64)
template <int FMT> struct WTile;
template <> struct WTile<FMT_Q4K> { static constexpr u32 SB = 144, PIECES = 9, DMA = 5, BYTES = 32 * 144; };
template <> struct WTile<FMT_Q5K> { static constexpr u32 SB = 176, PIECES = 11, DMA = 6, BYTES = 32 * 176; };
// dynamic LDS: two stages of token operands, two weight tiles per wave, one word for the arrival order
__host__ __device__ constexpr u32 lds_bytes(u32 waves, u32 tile_bytes, u32 nt) { return 2u * nt * kXpStageBytes + 2u * waves * tile_bytes + 16u; }

__device__ __forceinline__ u32 wave_max_u32(u32 v) {
  v = max(v, static_cast<u32>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0xB1, 0xF, 0xF, true)));
  v = max(v, static_cast<u32>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0x4E, 0xF, 0xF, true)));
  v = max(v, static_cast<u32>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0x141, 0xF, 0xF, true)));
  v = max(v, static_cast<u32>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0x140, 0xF, 0xF, true)));
  const u32 a = static_cast<u32>(__builtin_amdgcn_readlane(static_cast<int>(v), 0));
  const u32 b = static_cast<u32>(__builtin_amdgcn_readlane(static_cast<int>(v), 16));
  const u32 c = static_cast<u32>(__builtin_amdgcn_readlane(static_cast<int>(v), 32));
  const u32 d = static_cast<u32>(__builtin_amdgcn_readlane(static_cast<int>(v), 48));
  return max(max(a, b), max(c, d));
}

// hi and lo piece of a scaled value (|v| < 2^15, or not finite)
__device__ __forceinline__ void split_f16(float v, _Float16& hi, _Float16& lo) {
  hi = static_cast<_Float16>(v);
  lo = static_cast<_Float16>((v - static_cast<float>(hi)) * 2048.0f);
}

__device__ __forceinline__ u32 pack_h2(_Float16 a, _Float16 b) {
  const h16x2 p = {a, b};
  return __builtin_bit_cast(u32, p);
}

// ---- LDS through inline asm ----------------------------------------------------------------------
template <int OFF>
__device__ __forceinline__ void lds_read128(u32x4& v, u32 addr) {
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=&v"(v) : "v"(addr), "n"(OFF) : "memory");
}
template <int OFF>
__device__ __forceinline__ void lds_read64(u32x2& v, u32 addr) {
  asm volatile("ds_read_b64 %0, %1 offset:%2" : "=&v"(v) : "v"(addr), "n"(OFF) : "memory");
}
// waits for every LDS read issued so far; the values pass through so that no use moves above the wait
__device__ __forceinline__ void lds_wait4(u32x4& a, u32x4& b, u32x4& c, u32x4& d) {
  asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a), "+v"(b), "+v"(c), "+v"(d)::"memory");
}
__device__ __forceinline__ void lds_wait5(u32x4& a, u32x4& b, u32x4& c, u32x4& d, u32x4& e, u32x2& f) {
  asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a), "+v"(b), "+v"(c), "+v"(d), "+v"(e), "+v"(f)::"memory");
}

__device__ __forceinline__ void dma16(const uint8_t* src, u32 lds_addr) {
  __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                   (__attribute__((address_space(3))) void*)(uintptr_t)lds_addr, 16, 0, 0);
}

__device__ __forceinline__ void lds_write128x2(u32 addr, const u32x4& a, const u32x4& b) {
  asm volatile("ds_write_b128 %0, %1\n\tds_write_b128 %0, %2 offset:16" ::"v"(addr), "v"(a), "v"(b) : "memory");
}
template <int APART>
__device__ __forceinline__ void lds_write16x2(u32 addr, u32 a, u32 b) {     // the low halves of a and b, APART bytes apart
  asm volatile("ds_write_b16 %0, %1\n\tds_write_b16 %0, %2 offset:%3" ::"v"(addr), "v"(a), "v"(b), "n"(APART) : "memory");
}
__device__ __forceinline__ void lds_write32(u32 addr, u32 a) { asm volatile("ds_write_b32 %0, %1" ::"v"(addr), "v"(a) : "memory"); }

// Token operands of one super-block, written to an LDS stage of kXpStageBytes:
//   q*1024 + ((32g + 2*token + piece) ^ 2q)*16 + 2e   f16 = piece of the scaled element 32 j + 8 (u%4) + perm[e],
//                                               u = q/2, h = q%2, j = 2 (2g + u/4) + h, perm = 0,2,1,3,4,6,5,7
//   16384 + (32g + 2*token + piece)*8 + 2e     f16 = piece of 2^-5 * (sum of the scaled sub-block 4g + e)
//   16896 + token*4                            f32 = 2^(E+14) where the run was scaled by 2^-E (NaN if the run
//                                               holds an infinity or a NaN)
// This thread brings the eight elements 8c .. 8c+7 (v0, v1) of token `token` of the tile; the 32 threads of a
// half wave hold one token's run.
// SUMS = false (Q6_K, whose kernel needs no sums) leaves the sums out.
template <bool SUMS = true>
__device__ __forceinline__ void convert_chunk(const f32x4& v0, const f32x4& v1, u32 token, u32 c, u32 stage) {
  const u32 lane = threadIdx.x & 63u;
  const float x[8] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w};
  u32 amax = 0u;
#pragma unroll
  for (int e = 0; e < 8; ++e) amax = max(amax, __float_as_uint(x[e]) & 0x7FFFFFFFu);
  amax = max(amax, static_cast<u32>(__builtin_amdgcn_update_dpp(0, static_cast<int>(amax), 0xB1, 0xF, 0xF, true)));
  amax = max(amax, static_cast<u32>(__builtin_amdgcn_update_dpp(0, static_cast<int>(amax), 0x4E, 0xF, 0xF, true)));
  amax = max(amax, static_cast<u32>(__builtin_amdgcn_update_dpp(0, static_cast<int>(amax), 0x141, 0xF, 0xF, true)));
  amax = max(amax, static_cast<u32>(__builtin_amdgcn_update_dpp(0, static_cast<int>(amax), 0x140, 0xF, 0xF, true)));
  const u32 r0 = static_cast<u32>(__builtin_amdgcn_readlane(static_cast<int>(amax), 0));
  const u32 r1 = static_cast<u32>(__builtin_amdgcn_readlane(static_cast<int>(amax), 16));
  const u32 r2 = static_cast<u32>(__builtin_amdgcn_readlane(static_cast<int>(amax), 32));
  const u32 r3 = static_cast<u32>(__builtin_amdgcn_readlane(static_cast<int>(amax), 48));
  amax = lane < 32u ? max(r0, r1) : max(r2, r3);
  u32 eb = amax >> 23;                      // biased exponent of the run's maximum
  const bool finite = eb != 255u;
  eb = eb < 14u ? 14u : eb;                 // keeps both powers of two normal; a run that tiny loses nothing that matters
  const float down = __uint_as_float((268u - eb) << 23);        // 2^-E = 2^(141 - eb)
  _Float16 hi[8], lo[8];
  float xs[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    xs[e] = x[e] * down;
    split_f16(xs[e], hi[e], lo[e]);
  }
  const u32 j = c >> 2, g = j >> 2, h = j & 1u, u = 4u * ((j & 3u) >> 1) + (c & 3u), q = 2u * u + h;
  const u32x4 ph = {pack_h2(hi[0], hi[2]), pack_h2(hi[1], hi[3]), pack_h2(hi[4], hi[6]), pack_h2(hi[5], hi[7])};
  const u32x4 pl = {pack_h2(lo[0], lo[2]), pack_h2(lo[1], lo[3]), pack_h2(lo[4], lo[6]), pack_h2(lo[5], lo[7])};
  // the 16 products' pages are 1 KB apart, i.e. on the same banks: slot s of page q lies at s ^ 2q, so that the lanes
  // of a token, which write the same slot of different pages, do not all hit one bank (the reader applies the same)
  lds_write128x2(stage + q * 1024u + ((32u * g + 2u * token) ^ (2u * q)) * 16u, ph, pl);
  if constexpr (SUMS) {
    // The sub-block's sum is formed from the pieces, not from the f32 values: a piece has eleven significant bits, so
    // thirty-two of them of similar size add up without rounding in f32, where the values themselves round at every
    // step - and the sum is multiplied by C * s_j (the centring term of the Q4_K / Q5_K products), which is large.
    const h16x2 ones = {static_cast<_Float16>(1.0f), static_cast<_Float16>(1.0f)};
    float sh = __builtin_amdgcn_fdot2(as_h16x2(ph.x), ones, 0.0f, false), sl = __builtin_amdgcn_fdot2(as_h16x2(pl.x), ones, 0.0f, false);
    sh = __builtin_amdgcn_fdot2(as_h16x2(ph.y), ones, sh, false); sl = __builtin_amdgcn_fdot2(as_h16x2(pl.y), ones, sl, false);
    sh = __builtin_amdgcn_fdot2(as_h16x2(ph.z), ones, sh, false); sl = __builtin_amdgcn_fdot2(as_h16x2(pl.z), ones, sl, false);
    sh = __builtin_amdgcn_fdot2(as_h16x2(ph.w), ones, sh, false); sl = __builtin_amdgcn_fdot2(as_h16x2(pl.w), ones, sl, false);
    sh += dpp_f32<0xB1>(sh); sl += dpp_f32<0xB1>(sl);
    sh += dpp_f32<0x4E>(sh); sl += dpp_f32<0x4E>(sl);      // the four threads of a sub-block hold its sums
    const float sj = fmaf(sl, 0.00048828125f, sh);
    if ((c & 3u) == 0u) {
      _Float16 sh, sl;
      split_f16(sj * 0.03125f, sh, sl);
      lds_write16x2<8>(stage + kXpMainBytes + (32u * g + 2u * token) * 8u + 2u * (j & 3u), pack_h2(sh, sh), pack_h2(sl, sl));
    }
  }
  if (c == 0u) lds_write32(stage + kXpMainBytes + kXpSumBytes + 4u * token, finite ? (eb << 23) : 0x7FC00000u);
}

__device__ __forceinline__ h16x2 pk_mul_h2(u32 bits, h16x2 s) { return as_h16x2(bits) * s; }
__device__ __forceinline__ h16x2 pk_fma_h2(u32 bits, h16x2 s, h16x2 add) { return __builtin_elementwise_fma(as_h16x2(bits), s, add); }

constexpr u32 kCounterBytes = 1u << 16;        // arrival counters at the front of the workspace, the partial sums behind them

// What the kernels do with the finished tiles of a workgroup (NT token tiles of 16: tiles tg*NT .. tg*NT + NT - 1).
// lane l, tot registers 4a + 2b + piece: token 4a + 2g + b of the tile, W row strip*32 + col.  With one part of K the
// results are stored; otherwise the part is published and the workgroup that arrives last at the (group, tile group)
// counter adds the parts in part order - the sum does not depend on who is last - and puts the counter back to zero.
// (A counter per strip, each wave on its own without the two barriers, was measured 0.5-1 us slower: eight times as
// many atomic operations on neighbouring addresses.)
template <int NT>
__device__ __forceinline__ void finish_tiles(const f32x16 (&tot)[NT], float* __restrict__ c, uint8_t* __restrict__ ws,
                                             u32 m, u32 n, u32 kparts, u32 groups, u32 tiles, u32 tgroups, u32 waves, u32 group, u32 part,
                                             u32 tg, u32 strip, u32 col, u32 g, u32 lane, u32 lds_flag) {
  const u32 row = strip * 32u + col;
  const bool row_ok = row < n;
  float val[NT][8];
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
      for (int b = 0; b < 2; ++b) val[t][2 * a + b] = fmaf(tot[t][4 * a + 2 * b + 1], 0.00048828125f, tot[t][4 * a + 2 * b]);
  if (kparts == 1u) {
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int b = 0; b < 2; ++b) {
          const u32 token = (tg * NT + t) * kTokensPerTile + 4u * a + 2u * g + b;
          if (row_ok && token < m) c[static_cast<size_t>(token) * n + row] = val[t][2 * a + b];
        }
    return;
  }
  // The parts cross workgroups (and XCDs): 16-byte buffer accesses at agent scope (sc1); a wave's tokens 0..7 of the
  // tile as one KB (lane l at 16 l), its tokens 8..15 as the next, so that a store instruction writes whole lines:
  //   partial[((part * tiles + tile) * strips + strip)][2][64 lanes][4]
  u32* counters = reinterpret_cast<u32*>(ws);
  const u32 strips = groups * waves;
  const __amdgpu_buffer_rsrc_t part_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      ws + kCounterBytes, 0, static_cast<int>(static_cast<size_t>(kparts) * tiles * strips * 2048u), 0x00020000);
  auto slot_of = [&](u32 pt, u32 tile) { return static_cast<int>(((pt * tiles + tile) * strips + strip) * 2048u + lane * 16u); };
  bool lower[NT], upper[NT];      // tokens 0..7 / 8..15 of the tile exist (val[0..3] / val[4..7])
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const u32 tile = tg * NT + t;
    lower[t] = tile * kTokensPerTile < m;
    upper[t] = tile * kTokensPerTile + 8u < m;
    if (lower[t])
      __builtin_amdgcn_raw_buffer_store_b128(u32x4{__float_as_uint(val[t][0]), __float_as_uint(val[t][1]), __float_as_uint(val[t][2]), __float_as_uint(val[t][3])},
                                             part_rsrc, slot_of(part, tile), 0, 16);
    if (upper[t])
      __builtin_amdgcn_raw_buffer_store_b128(u32x4{__float_as_uint(val[t][4]), __float_as_uint(val[t][5]), __float_as_uint(val[t][6]), __float_as_uint(val[t][7])},
                                             part_rsrc, slot_of(part, tile) + 1024, 0, 16);
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");      // the coherent stores have been acknowledged
  asm volatile("s_barrier" ::: "memory");
  if (threadIdx.x == 0u) {
    const u32 old = __hip_atomic_fetch_add(counters + group * tgroups + tg, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    asm volatile("ds_write_b32 %0, %1\n\ts_waitcnt lgkmcnt(0)" ::"v"(lds_flag), "v"(old) : "memory");
  }
  asm volatile("s_barrier" ::: "memory");
  u32 old;
  asm volatile("ds_read_b32 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(old) : "v"(lds_flag) : "memory");
  if (old == kparts - 1u && threadIdx.x == 0u)      // ready for the next product on this stream
    __hip_atomic_store(counters + group * tgroups + tg, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  if (old != kparts - 1u || !row_ok) return;
  float r[NT][8];
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int e = 0; e < 8; ++e) r[t][e] = 0.0f;
  // all parts in flight at once when they are few (a round trip to memory each time otherwise), added in part order;
  // no more loads than there are parts to the next power of two
  auto add_parts = [&](auto width) {
    constexpr u32 W = decltype(width)::value;
    for (u32 p0 = 0; p0 < kparts; p0 += W) {
      u32x4 lo[NT][W], hi[NT][W];
#pragma unroll
      for (int t = 0; t < NT; ++t)
#pragma unroll
        for (u32 pp = 0; pp < W; ++pp) {
          const u32 pt = min(p0 + pp, kparts - 1u);
          lo[t][pp] = lower[t] ? __builtin_amdgcn_raw_buffer_load_b128(part_rsrc, slot_of(pt, tg * NT + t), 0, 16) : u32x4{0u, 0u, 0u, 0u};
          hi[t][pp] = upper[t] ? __builtin_amdgcn_raw_buffer_load_b128(part_rsrc, slot_of(pt, tg * NT + t) + 1024, 0, 16) : u32x4{0u, 0u, 0u, 0u};
        }
#pragma unroll
      for (int t = 0; t < NT; ++t)
#pragma unroll
        for (u32 pp = 0; pp < W; ++pp)
          if (p0 + pp < kparts) {
            r[t][0] += __uint_as_float(lo[t][pp].x); r[t][1] += __uint_as_float(lo[t][pp].y); r[t][2] += __uint_as_float(lo[t][pp].z); r[t][3] += __uint_as_float(lo[t][pp].w);
            r[t][4] += __uint_as_float(hi[t][pp].x); r[t][5] += __uint_as_float(hi[t][pp].y); r[t][6] += __uint_as_float(hi[t][pp].z); r[t][7] += __uint_as_float(hi[t][pp].w);
          }
    }
  };
  if (kparts <= 2u) add_parts(std::integral_constant<u32, 2>{});
  else if (kparts <= 4u) add_parts(std::integral_constant<u32, 4>{});
  else if (kparts <= 8u || NT > 1) add_parts(std::integral_constant<u32, 8>{});
  else add_parts(std::integral_constant<u32, 16>{});
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const u32 token = (tg * NT + t) * kTokensPerTile + 4u * (e >> 1) + 2u * g + (e & 1);
      if (token < m) c[static_cast<size_t>(token) * n + row] = r[t][e];
    }
}

// What every kernel of this file takes: the operands, the workspace (counters, then partial sums), the shape and
// the cut - geom = ksb | kparts << 16 | groups << 32 | tiles << 48 - in eight arguments, which the hardware hands
// over in registers at the start of a wave (kernel-argument preload), so that nothing is read before the first loads.
struct Geometry {
  u32 ksb, kparts, groups, tiles;
  __device__ explicit Geometry(uint64_t geom)
      : ksb(static_cast<u32>(geom) & 0xFFFFu), kparts(static_cast<u32>(geom >> 16) & 0xFFFFu),
        groups(static_cast<u32>(geom >> 32) & 0xFFFFu), tiles(static_cast<u32>(geom >> 48)) {}
};

// Main kernel.  Workgroup id -> (unit, tile group) with the tile groups of a unit 8 ids apart (same XCD, so the
// weights they share meet in that XCD's L2); unit -> (group of 8 strips, part of K).  A workgroup takes NT token
// tiles (a tile group): the weight operands of a product are built once and meet NT tiles' tokens, which is what
// pays when the tokens are many - building them is most of a super-block's instructions.  (finish_tiles: what
// happens with the results.)
//   dynamic LDS = lds_bytes(waves, tile bytes, NT)
template <int FMT, int WAVES, int NT>     // WAVES strips of 32 rows per workgroup (4, 8 or 12): the kernels are launched with 64 * WAVES threads
__device__ __forceinline__ void kq_body(const float* __restrict__ a, const uint8_t* __restrict__ w, float* __restrict__ c, uint8_t* __restrict__ ws,
                                         u32 m, u32 n, u32 nsb, uint64_t geom, u32 lds_base) {
  const Geometry cut(geom);
  const u32 ksb = cut.ksb, kparts = cut.kparts, groups = cut.groups, tiles = cut.tiles;
  const u32 lane = threadIdx.x & 63u;
  const u32 wave = static_cast<u32>(__builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x >> 6)));
  const u32 id = blockIdx.x;
  const u32 tgroups = (tiles + NT - 1u) / NT;
  const u32 unit = (id / (8u * tgroups)) * 8u + (id & 7u), tg = (id >> 3) % tgroups;
  if (unit >= groups * kparts) return;
  const u32 group = unit / kparts, part = unit - group * kparts;
  const u32 sb0 = part * ksb, ns = min(ksb, nsb - sb0);
  constexpr u32 waves = WAVES;
  // chunks of A a thread converts per super-block and tile: 512 over the threads (with 12 waves the last four convert none)
  constexpr int CHUNKS = WAVES >= 8 ? 1 : 8 / WAVES;
  const u32 strip = group * waves + wave;
  const u32 col = lane & 31u, g = lane >> 5;
  using T = WTile<FMT>;
  constexpr u32 kWStageBytes = T::BYTES;
  constexpr int DMA = static_cast<int>(T::DMA);
  const size_t row_bytes = static_cast<size_t>(nsb) * T::SB;

  // where this lane's pieces of a weight tile come from: piece p = 64 t + lane of [32 rows][PIECES pieces]
  size_t woff[DMA];
#pragma unroll
  for (int t = 0; t < DMA; ++t) {
    const u32 p = min(64u * t + lane, 32u * T::PIECES - 1u);
    const u32 r = p / T::PIECES, cc = p - T::PIECES * r;
    woff[t] = static_cast<size_t>(min(strip * 32u + r, n - 1u)) * row_bytes + 16u * cc;
  }
  constexpr u32 kStage = NT * kXpStageBytes;      // the token operands of one super-block: NT tiles one behind the other
  const u32 lds_xp = lds_base, lds_w = lds_base + 2u * kStage + wave * (2u * kWStageBytes);
  const u32 lds_flag = lds_base + 2u * kStage + 2u * waves * kWStageBytes;
  // the chunks of A this thread converts per super-block: 512 chunks of 8 elements (16 tokens x 32)
  constexpr u32 nthreads = 64u * WAVES;
  constexpr int NC = CHUNKS * NT;      // chunk i: tile i / CHUNKS of the group
  const bool converts = WAVES <= 8 || wave < 8u;      // (the others load the same A all the same: one count of loads for every wave)
  const float* asrc[NC];
  u32 ctoken[NC], cpos[NC];
  bool live[NC];
#pragma unroll
  for (int i = 0; i < NC; ++i) {
    const u32 idx = threadIdx.x + (i % CHUNKS) * nthreads;
    ctoken[i] = (idx >> 5) & 15u;
    cpos[i] = idx & 31u;
    const u32 token = (tg * NT + i / CHUNKS) * kTokensPerTile + ctoken[i];
    asrc[i] = a + static_cast<size_t>(min(token, m - 1u)) * (static_cast<size_t>(nsb) * 256u) + 8u * cpos[i];
    live[i] = token < m;
  }

  // Loads are counted by hand (s_waitcnt vmcnt): per super-block a wave issues 2*NC loads of A, then DMA of W.  (With
  // ordinary loads of A the compiler waits for vmcnt(0) wherever DMA is also in flight, which takes the copies of W out
  // of the background.  The price of asm: between such a load and the wait that names its registers the compiler must
  // have no reason to copy them - one definition per loop, no second set of registers joined to the first; a variant
  // that requested two super-blocks up front broke exactly there; the build refuses such assembly (check_asm_loads.py) and
  // the parity tests show it at once.)
  auto issue_w = [&](u32 s) {
    const uint8_t* wsrc = w + static_cast<size_t>(sb0 + s) * T::SB;
    const u32 wl = lds_w + (s & 1u) * kWStageBytes;
#pragma unroll
    for (int t = 0; t < DMA - 1; ++t) dma16(wsrc + woff[t], wl + 1024u * t);
    if (lane < 32u) dma16(wsrc + woff[DMA - 1], wl + 1024u * (DMA - 1));
  };
  u32x4 an[NC][2];                     // A of a super-block on its way to conversion
  auto load_a = [&](u32 s) {
#pragma unroll
    for (int i = 0; i < NC; ++i) {
      const float* src = asrc[i] + static_cast<size_t>(sb0 + s) * 256u;
      asm volatile("global_load_dwordx4 %0, %2, off\n\tglobal_load_dwordx4 %1, %2, off offset:16"
                   : "=&v"(an[i][0]), "=&v"(an[i][1]) : "v"(src) : "memory");
    }
  };
  // The loads of A issued last have landed when no more than the copies of W behind them are outstanding.  The last of
  // those copies stands under `lane < 32`, which the compiler turns into a branch around it: on paper a wave can pass
  // with DMA - 1 copies behind its loads of A, so that is the number waited for (it costs the first sixteenth of the
  // weight tile having arrived as well).
  auto convert = [&](u32 s) {
#pragma unroll
    for (int i = 0; i < NC; ++i) asm volatile("s_waitcnt vmcnt(%2)" : "+v"(an[i][0]), "+v"(an[i][1]) : "n"(DMA - 1) : "memory");
    const f32x4 zero4 = {0.0f, 0.0f, 0.0f, 0.0f};
    if (!converts) return;
#pragma unroll
    for (int i = 0; i < NC; ++i)
      convert_chunk(live[i] ? __builtin_bit_cast(f32x4, an[i][0]) : zero4, live[i] ? __builtin_bit_cast(f32x4, an[i][1]) : zero4,
                    ctoken[i], cpos[i], lds_xp + (s & 1u) * kStage + (i / CHUNKS) * kXpStageBytes);
  };

  // Two running sums per result, for the even and the odd super-blocks of the run: each is half as long and half as
  // large when it is rounded as one sum over all of them would be (the reference spreads a row over 32 lanes' sums,
  // quantize.rs:1486, 1495-1508; here one register holds a whole row's).
  f32x16 tot[NT], tot_odd[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int v = 0; v < 16; ++v) tot[t][v] = tot_odd[t][v] = 0.0f;
  u32 xq[16];                                    // where this lane finds its token operands of product q (stage 0)
#pragma unroll
  for (u32 q = 0; q < 16; ++q) xq[q] = lds_xp + ((lane ^ (2u * q)) << 4);

  load_a(0);
  issue_w(0);
  convert(0);
  if (ns > 1u) {
    load_a(1);
    issue_w(1);
  }
  for (u32 s = 0; s < ns; ++s) {
    // weight tile s has landed (the loads of super-block s+1 may be in flight); the token operands of s are written
    if (s + 1u < ns) asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(2 * NC + DMA) : "memory");
    else asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    asm volatile("s_barrier" ::: "memory");
    const u32 slot = s & 1u;
    const u32 wt = lds_w + slot * kWStageBytes + col * T::SB, wl = wt + g * 64u;
    const u32 sl = lds_xp + slot * kStage + kXpMainBytes + lane * 8u;
    const u32 fl = lds_xp + slot * kStage + kXpMainBytes + kXpSumBytes + g * 8u;
    u32x4 hdr, d0, d1, d2, d3;
    u32x2 sx[NT], f01[NT], f23[NT], f45[NT], f67[NT];
    asm volatile("ds_read_b128 %0, %1" : "=&v"(hdr) : "v"(wt) : "memory");
    lds_read128<16>(d0, wl);
    lds_read128<32>(d1, wl);
    lds_read128<48>(d2, wl);
    lds_read128<64>(d3, wl);
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      lds_read64<0>(sx[t], sl + t * kXpStageBytes);
      lds_read64<0>(f01[t], fl + t * kXpStageBytes);          // 2^(E+14) of the tokens 4a + 2g + {0, 1}, a = 0..3
      lds_read64<16>(f23[t], fl + t * kXpStageBytes);
      lds_read64<32>(f45[t], fl + t * kXpStageBytes);
      lds_read64<48>(f67[t], fl + t * kXpStageBytes);
    }
    [[maybe_unused]] u32x4 qh = {0u, 0u, 0u, 0u};      // Q5_K: this lane group's 16 bytes of fifth bits (values 128 g .. 128 g + 127)
    if constexpr (FMT == FMT_Q5K) lds_read128<144>(qh, wt + g * 16u);
    lds_wait5(hdr, d0, d1, d2, d3, sx[0]);
#pragma unroll
    for (int t = 0; t < NT; ++t) asm volatile("" : "+v"(sx[t]), "+v"(f01[t]), "+v"(f23[t]), "+v"(f45[t]), "+v"(f67[t]));
    asm volatile("" : "+v"(qh));
    if (s + 1u < ns) {
      convert(s + 1u);          // into the stage that was read two super-blocks ago
      if (s + 2u < ns) {        // the weight tile is in registers: its LDS space takes the tile after the next
        load_a(s + 2u);         // (inside the first condition: no path issues loads without having waited for the last ones)
        issue_w(s + 2u);
      }
    }
    const u32 dw[16] = {d0.x, d0.y, d0.z, d0.w, d1.x, d1.y, d1.z, d1.w, d2.x, d2.y, d2.z, d2.w, d3.x, d3.y, d3.z, d3.w};
    const float d = half_bits_to_f32(hdr.x), dmin = half_bits_to_f32(hdr.x >> 16);
    // this lane's four 6-bit scales and mins (sub-blocks 4g .. 4g+3) as bytes
    u32 s4, m4;
    if constexpr (FMT == FMT_Q4K) {      // get_scale_min_k4, quantize.rs:1306-1385
      s4 = g ? ((hdr.w & 0x0F0F0F0Fu) | ((hdr.y >> 2) & 0x30303030u)) : (hdr.y & 0x3F3F3F3Fu);
      m4 = g ? (((hdr.w >> 4) & 0x0F0F0F0Fu) | ((hdr.z >> 2) & 0x30303030u)) : (hdr.z & 0x3F3F3F3Fu);
    } else {                             // eight contiguous 12-bit fields, scale in the low six bits (quantize.rs:1607-1635)
      const u32 lo = g ? ((hdr.z >> 16) | (hdr.w << 16)) : hdr.y;      // fields 4g, 4g+1 and the low byte of 4g+2
      const u32 hi = g ? (hdr.w >> 16) : (hdr.z & 0xFFFFu);            // the rest of field 4g+2 and field 4g+3
      const u32 f0 = lo & 0xFFFu, f1 = (lo >> 12) & 0xFFFu, f2 = ((lo >> 24) | (hi << 8)) & 0xFFFu, f3 = (hi >> 4) & 0xFFFu;
      s4 = (f0 & 63u) | ((f1 & 63u) << 8) | ((f2 & 63u) << 16) | ((f3 & 63u) << 24);
      m4 = (f0 >> 6) | ((f1 >> 6) << 8) | ((f2 >> 6) << 16) | ((f3 >> 6) << 24);
    }
    // The quants enter centred: (q - C) * s_j with C = 8 (Q4_K) or 16 (Q5_K), and C * s_j * (sum of the sub-block's
    // activations) is added by one small product at the end.  The running sums inside the matrix cores are then those of
    // numbers spread around zero, about half as large as with q >= 0, and so are their rounding errors (measured:
    // 1.2 times the error of an f32 evaluation in the reference's order uncentred; Q6_K, whose digits are centred by
    // construction, 1.0).  (q - C) * s_j stays below 2048 in magnitude: exact in f16, as is the multiply-add that forms it.
    constexpr float kCentre = FMT == FMT_Q4K ? 8.0f : 16.0f;
    h16x2 sc[4], ad[4];
    _Float16 sf[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      sf[e] = static_cast<_Float16>(static_cast<unsigned short>((s4 >> (8 * e)) & 0xFFu));
      const _Float16 sv = sf[e] * static_cast<_Float16>((e & 1) ? 64.0f : 1024.0f);
      const _Float16 av = sf[e] * static_cast<_Float16>(-kCentre * 0.00006103515625f);      // -C * s_j * 2^-14
      sc[e] = h16x2{sv, sv};
      ad[e] = h16x2{av, av};
    }
    // C * s_j * 2^-9 against the sub-block sums (which carry 2^-5): C * s_j * 2^-14 * sum, the scale of the main products
    const h16x4 cb = {sf[0] * static_cast<_Float16>(kCentre * 0.001953125f), sf[1] * static_cast<_Float16>(kCentre * 0.001953125f),
                      sf[2] * static_cast<_Float16>(kCentre * 0.001953125f), sf[3] * static_cast<_Float16>(kCentre * 0.001953125f)};
    const h16x4 mb = {static_cast<_Float16>(static_cast<unsigned short>(m4 & 0xFFu)),
                      static_cast<_Float16>(static_cast<unsigned short>((m4 >> 8) & 0xFFu)),
                      static_cast<_Float16>(static_cast<unsigned short>((m4 >> 16) & 0xFFu)),
                      static_cast<_Float16>(static_cast<unsigned short>(m4 >> 24))};
    const f32x16 zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    f32x16 macc[NT], acc[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) acc[t] = zero;
#pragma unroll
    for (int uu = 0; uu < 8; uu += 2) {          // two dword pairs = four products per round of operand reads
      u32x4 ax[NT][4];
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        const u32 xs = slot * kStage + t * kXpStageBytes;       // product q reads slot lane ^ 2q of its page (xq[q], set up once)
        switch (uu) {
          case 0: lds_read128<0 * 1024>(ax[t][0], xq[0] + xs); lds_read128<1 * 1024>(ax[t][1], xq[1] + xs); lds_read128<2 * 1024>(ax[t][2], xq[2] + xs); lds_read128<3 * 1024>(ax[t][3], xq[3] + xs); break;
          case 2: lds_read128<4 * 1024>(ax[t][0], xq[4] + xs); lds_read128<5 * 1024>(ax[t][1], xq[5] + xs); lds_read128<6 * 1024>(ax[t][2], xq[6] + xs); lds_read128<7 * 1024>(ax[t][3], xq[7] + xs); break;
          case 4: lds_read128<8 * 1024>(ax[t][0], xq[8] + xs); lds_read128<9 * 1024>(ax[t][1], xq[9] + xs); lds_read128<10 * 1024>(ax[t][2], xq[10] + xs); lds_read128<11 * 1024>(ax[t][3], xq[11] + xs); break;
          default: lds_read128<12 * 1024>(ax[t][0], xq[12] + xs); lds_read128<13 * 1024>(ax[t][1], xq[13] + xs); lds_read128<14 * 1024>(ax[t][2], xq[14] + xs); lds_read128<15 * 1024>(ax[t][3], xq[15] + xs); break;
        }
      }
      u32 bl[2][4], bh[2][4];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int u = uu + i;
        const u32 t0 = dw[2 * u], t1 = dw[2 * u + 1], t0s = t0 >> 8, t1s = t1 >> 8;
        const h16x2 sl2 = sc[(u >> 2) * 2], sh2 = sc[(u >> 2) * 2 + 1], al2 = ad[(u >> 2) * 2], ah2 = ad[(u >> 2) * 2 + 1];
        // Q5_K: the fifth bits of the eight values of dword j (j = 2u, 2u+1) are nibble j%8 of qh word 2(j/8) (low
        // nibbles) and 2(j/8)+1 (high nibbles), bit i for byte i.  n * (2^4 + 2^18) puts bit 0 at bit 4 and bit 2 at
        // bit 20 - where the fifth bit of a low nibble's 16-bit lane belongs for bytes 0 and 2 -, n * (2^3 + 2^17) the
        // same for bytes 1 and 3; for the high nibbles (quant in bits 4..7 of its lane) four places further up.
        u32 f[2][4] = {{0u, 0u, 0u, 0u}, {0u, 0u, 0u, 0u}}, e[2][4] = {{0u, 0u, 0u, 0u}, {0u, 0u, 0u, 0u}};
        if constexpr (FMT == FMT_Q5K) {
          const u32 ql5 = u < 4 ? qh.x : qh.z, qh5 = u < 4 ? qh.y : qh.w;
#pragma unroll
          for (int d = 0; d < 2; ++d) {
            const u32 nl = (ql5 >> (4 * ((2 * u + d) & 7))) & 15u, nh = (qh5 >> (4 * ((2 * u + d) & 7))) & 15u;
            f[d][0] = __umul24(nl, 0x40010u) & 0x00100010u;      // low nibbles, bytes 0 and 2
            f[d][1] = __umul24(nl, 0x20008u) & 0x00100010u;      // low nibbles, bytes 1 and 3
            e[d][0] = __umul24(nh, 0x400100u) & 0x01000100u;     // high nibbles, bytes 0 and 2
            e[d][1] = __umul24(nh, 0x200080u) & 0x01000100u;     // high nibbles, bytes 1 and 3
          }
        }
        bl[i][0] = __builtin_bit_cast(u32, pk_fma_h2((t0 & 0x000F000Fu) | f[0][0], sl2, al2));
        bl[i][1] = __builtin_bit_cast(u32, pk_fma_h2((t0s & 0x000F000Fu) | f[0][1], sl2, al2));
        bl[i][2] = __builtin_bit_cast(u32, pk_fma_h2((t1 & 0x000F000Fu) | f[1][0], sl2, al2));
        bl[i][3] = __builtin_bit_cast(u32, pk_fma_h2((t1s & 0x000F000Fu) | f[1][1], sl2, al2));
        bh[i][0] = __builtin_bit_cast(u32, pk_fma_h2((t0 & 0x00F000F0u) | e[0][0], sh2, ah2));
        bh[i][1] = __builtin_bit_cast(u32, pk_fma_h2((t0s & 0x00F000F0u) | e[0][1], sh2, ah2));
        bh[i][2] = __builtin_bit_cast(u32, pk_fma_h2((t1 & 0x00F000F0u) | e[1][0], sh2, ah2));
        bh[i][3] = __builtin_bit_cast(u32, pk_fma_h2((t1s & 0x00F000F0u) | e[1][1], sh2, ah2));
      }
#pragma unroll
      for (int t = 0; t < NT; ++t) lds_wait4(ax[t][0], ax[t][1], ax[t][2], ax[t][3]);
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const u32x4 blv = {bl[i][0], bl[i][1], bl[i][2], bl[i][3]}, bhv = {bh[i][0], bh[i][1], bh[i][2], bh[i][3]};
#pragma unroll
        for (int t = 0; t < NT; ++t)
          acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(h16x8, ax[t][2 * i]), __builtin_bit_cast(h16x8, blv), acc[t], 0, 0, 0);
#pragma unroll
        for (int t = 0; t < NT; ++t)
          acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(h16x8, ax[t][2 * i + 1]), __builtin_bit_cast(h16x8, bhv), acc[t], 0, 0, 0);
      }
    }
    // what the centring took out, added to the main products in one step; then the min term's product (last: its
    // sixteen results per tile are not alive while the main products run)
#pragma unroll
    for (int t = 0; t < NT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_32x32x8f16(__builtin_bit_cast(h16x4, sx[t]), cb, acc[t], 0, 0, 0);
#pragma unroll
    for (int t = 0; t < NT; ++t) macc[t] = __builtin_amdgcn_mfma_f32_32x32x8f16(__builtin_bit_cast(h16x4, sx[t]), mb, zero, 0, 0, 0);
    const float nm = dmin * -0.001953125f;       // -dmin * 2^-9: the sums carry 2^-5, the products 2^-14
    // the super-block's own term is formed first (it is small), then added: one rounding at the size of the running sum
    // and the two running sums change places, so that each takes every other super-block
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      const float fac[8] = {__uint_as_float(f01[t].x), __uint_as_float(f01[t].y), __uint_as_float(f23[t].x), __uint_as_float(f23[t].y),
                            __uint_as_float(f45[t].x), __uint_as_float(f45[t].y), __uint_as_float(f67[t].x), __uint_as_float(f67[t].y)};
      const f32x16 other = tot[t];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float fd = fac[e] * d, fm = fac[e] * nm;
        tot[t][2 * e] = tot_odd[t][2 * e] + fmaf(fm, macc[t][2 * e], fd * acc[t][2 * e]);
        tot[t][2 * e + 1] = tot_odd[t][2 * e + 1] + fmaf(fm, macc[t][2 * e + 1], fd * acc[t][2 * e + 1]);
      }
      tot_odd[t] = other;
    }
  }
  // nothing is outstanding here (the last round waited for everything); said once more for the code that follows, which
  // takes over the registers of the loads written in asm
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
  for (int t = 0; t < NT; ++t) tot[t] += tot_odd[t];

  finish_tiles<NT>(tot, c, ws, m, n, kparts, groups, tiles, tgroups, waves, group, part, tg, strip, col, g, lane, lds_flag);
}


// ------------------------------------------------------------------------------------------------------------
// Q6_K (quantize.rs:1806-1934: ql[128] @0, qh[64] @128, sc[16] int8 @192, d f16 @208; w = d * sc * (q - 32) with
// q = nibble | (two bits of qh) << 4, scales per 16 values) on the matrix cores.
//   * (q - 32) * sc needs 13 bits: not exact in f16.  With centred digits  q - 32 = (nib - 8) + 8 (2 q2 - 3)  the two
//     products (nib - 8) sc (at most 8 * 128) and (2 q2 - 3) sc (at most 3 * 128) are exact operands, neither is large
//     against the value they add up to, and no sum of the tokens is needed.  Both come from the bits in place as for
//     Q4_K: a nibble or a 2-bit field moved to bits 4..7 of its 16-bit lane is the subnormal v * 2^-20; one packed
//     multiply-add with (sc * 2^6, -8 sc * 2^-14), or (sc * 2^7, -3 sc * 2^-14), gives the operand times 2^-14.  Two
//     accumulators over the super-block are combined per (row, token, super-block):  tot += d * 2^E * (acc_n + 8 acc_q).
//   * lane group g = l/32 of W row r takes half g of the super-block (values 128g .. 128g+127: ql[64g ..], qh[32g ..],
//     sc[8g ..]).  Token page Q of the Q4_K layout (values 128g + 64(U/4) + 32(Q%2) + 8(U%4) + .., U = Q/2) holds the
//     eight values that the low (U/4 = 0) or high nibbles of ql dwords 8(Q%2) + 2(U%4) + {0, 1} and field 2(U/4) + Q%2 of
//     qh dwords 2(U%4) + {0, 1} belong to: one read of a token page feeds two products.
//   * blocks of 210 bytes are only 2-byte aligned, which the copy into LDS by DMA does not take: the weight tile of
//     the NEXT super-block travels through registers (13 sixteen-byte loads and one 2-byte load per row, issued a
//     super-block ahead, written to LDS when the current one's products are done; rows 240 bytes apart in LDS, 15 pieces).
// Everything else (token conversion, parts of K, the sum over the parts) is the Q4_K kernel's.
constexpr u32 kQ6RowStride = 240u;                         // LDS bytes between the rows of a weight tile
constexpr u32 kQ6TileBytes = 32u * kQ6RowStride;
__host__ __device__ constexpr u32 q6k_lds_bytes(u32 waves) { return 2u * kXpStageBytes + waves * kQ6TileBytes + 16u; }

template <int CHUNKS>
__device__ __forceinline__ void q6k_body(const float* __restrict__ a, const uint8_t* __restrict__ w, float* __restrict__ c, uint8_t* __restrict__ ws,
                                         u32 m, u32 n, u32 nsb, uint64_t geom, u32 lds_base) {
  const Geometry cut(geom);
  const u32 ksb = cut.ksb, kparts = cut.kparts, groups = cut.groups, tiles = cut.tiles;
  const u32 lane = threadIdx.x & 63u;
  const u32 wave = static_cast<u32>(__builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x >> 6)));
  const u32 id = blockIdx.x;
  const u32 unit = (id / (8u * tiles)) * 8u + (id & 7u), tile = (id >> 3) % tiles;
  if (unit >= groups * kparts) return;
  const u32 group = unit / kparts, part = unit - group * kparts;
  const u32 sb0 = part * ksb, ns = min(ksb, nsb - sb0);
  constexpr u32 waves = 8u / CHUNKS;      // the kernels are launched with 512 / CHUNKS threads
  const u32 strip = group * waves + wave;
  const u32 col = lane & 31u, g = lane >> 5;
  const size_t row_bytes = static_cast<size_t>(nsb) * 210u;

  // this lane's pieces of a weight tile: piece p = 64 t + lane of [32 rows][13 pieces] (416 = 6.5 x 64), and the
  // row's last two bytes (d) by lanes 0..31
  size_t woff[7];
  u32 wdst[7];
#pragma unroll
  for (int t = 0; t < 7; ++t) {
    const u32 p = min(64u * t + lane, 415u);
    const u32 r = p / 13u, cc = p - 13u * r;
    woff[t] = static_cast<size_t>(min(strip * 32u + r, n - 1u)) * row_bytes + 16u * cc;
    wdst[t] = r * kQ6RowStride + 16u * cc;
  }
  const size_t doff = static_cast<size_t>(min(strip * 32u + col, n - 1u)) * row_bytes + 208u;
  const u32 lds_xp = lds_base, lds_w = lds_base + 2u * kXpStageBytes + wave * kQ6TileBytes;
  const u32 lds_flag = lds_base + 2u * kXpStageBytes + waves * kQ6TileBytes;
  constexpr u32 nthreads = 512u / CHUNKS;
  const float* asrc[CHUNKS];
  u32 ctoken[CHUNKS], cpos[CHUNKS];
  bool live[CHUNKS];
#pragma unroll
  for (int i = 0; i < CHUNKS; ++i) {
    const u32 idx = threadIdx.x + i * nthreads;
    ctoken[i] = (idx >> 5) & 15u;
    cpos[i] = idx & 31u;
    const u32 token = tile * kTokensPerTile + ctoken[i];
    asrc[i] = a + static_cast<size_t>(min(token, m - 1u)) * (static_cast<size_t>(nsb) * 256u) + 8u * cpos[i];
    live[i] = token < m;
  }

  // The loads of this kernel are ordinary ones and the compiler places the waits: values that stay in registers from
  // one super-block to the next and meet at the joins of the loop are copied where the compiler sees fit, which it may
  // only do with data that has arrived if it knows the load.  (The LDS side is written out by hand as in the Q4_K kernel.)
  u32x4 wn[7];                         // the next super-block's weight tile on its way to LDS
  u32 wd;
  auto load_w = [&](u32 s) {
    const uint8_t* wsrc = w + static_cast<size_t>(sb0 + s) * 210u;
#pragma unroll
    for (int t = 0; t < 7; ++t) wn[t] = load128_a2(wsrc + woff[t]);
    wd = load16_a2(wsrc + doff);
  };
  auto store_w = [&]() {
#pragma unroll
    for (int t = 0; t < 6; ++t) asm volatile("ds_write_b128 %0, %1" ::"v"(lds_w + wdst[t]), "v"(wn[t]) : "memory");
    if (lane < 32u) {
      asm volatile("ds_write_b128 %0, %1" ::"v"(lds_w + wdst[6]), "v"(wn[6]) : "memory");
      asm volatile("ds_write_b16 %0, %1" ::"v"(lds_w + col * kQ6RowStride + 208u), "v"(wd) : "memory");
    }
  };
  f32x4 an[CHUNKS][2];
  auto load_a = [&](u32 s) {
#pragma unroll
    for (int i = 0; i < CHUNKS; ++i) {
      const f32x4* src = reinterpret_cast<const f32x4*>(asrc[i] + static_cast<size_t>(sb0 + s) * 256u);
      an[i][0] = src[0];
      an[i][1] = src[1];
    }
  };
  auto convert = [&](u32 s) {
    const f32x4 zero4 = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int i = 0; i < CHUNKS; ++i)
      convert_chunk<false>(live[i] ? an[i][0] : zero4, live[i] ? an[i][1] : zero4, ctoken[i], cpos[i], lds_xp + (s & 1u) * kXpStageBytes);
  };

  // running sums over the even and the odd super-blocks (as in kq_body) where the registers allow it: the kernel of 4
  // strips converts twice the tokens per thread and is at the limit of two waves per SIMD with one sum
  constexpr bool kTwoSums = CHUNKS == 1;
  f32x16 tot, tot_odd;
#pragma unroll
  for (int v = 0; v < 16; ++v) tot[v] = tot_odd[v] = 0.0f;
  u32 xq[16];                                    // where this lane finds its token operands of page Q (stage 0)
#pragma unroll
  for (u32 q = 0; q < 16; ++q) xq[q] = lds_xp + ((lane ^ (2u * q)) << 4);

  // One super-block.  NEXT / NEXT2: super-blocks s+1 / s+2 exist (compile-time, so that every load is unconditional
  // where it stands: the loop below is peeled at its end).
  auto step = [&](u32 s, auto next_c, auto next2_c) {
    constexpr bool NEXT = decltype(next_c)::value, NEXT2 = decltype(next2_c)::value;
    // tile s is in LDS (this wave wrote it), the token operands of s are written by everybody
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    const u32 slot = s & 1u;
    const u32 wt = lds_w + col * kQ6RowStride;
    const u32 fl = lds_xp + slot * kXpStageBytes + kXpMainBytes + kXpSumBytes + g * 8u;
    u32x4 l0, l1, l2, l3, h0, h1;
    u32x2 scv, f01, f23, f45, f67;
    u32 dv;
    lds_read128<0>(l0, wt + g * 64u);
    lds_read128<16>(l1, wt + g * 64u);
    lds_read128<32>(l2, wt + g * 64u);
    lds_read128<48>(l3, wt + g * 64u);
    lds_read128<128>(h0, wt + g * 32u);
    lds_read128<144>(h1, wt + g * 32u);
    lds_read64<192>(scv, wt + g * 8u);
    asm volatile("ds_read_u16 %0, %1 offset:208" : "=&v"(dv) : "v"(wt) : "memory");
    lds_read64<0>(f01, fl);          // 2^(E+14) of the tokens 4a + 2g + {0, 1}, a = 0..3
    lds_read64<16>(f23, fl);
    lds_read64<32>(f45, fl);
    lds_read64<48>(f67, fl);
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(l0), "+v"(l1), "+v"(l2), "+v"(l3), "+v"(h0), "+v"(h1), "+v"(scv), "+v"(dv)::"memory");
    asm volatile("" : "+v"(f01), "+v"(f23), "+v"(f45), "+v"(f67));
    if constexpr (NEXT) convert(s + 1u);     // into the stage that was read two super-blocks ago
    if constexpr (NEXT2) load_a(s + 2u);
    const u32 ql[16] = {l0.x, l0.y, l0.z, l0.w, l1.x, l1.y, l1.z, l1.w, l2.x, l2.y, l2.z, l2.w, l3.x, l3.y, l3.z, l3.w};
    const u32 qh[8] = {h0.x, h0.y, h0.z, h0.w, h1.x, h1.y, h1.z, h1.w};
    const float d = half_bits_to_f32(dv);
    // this lane's eight int8 scales (sub-blocks 8g .. 8g+7) as the factors and addends of the two multiply-adds, each
    // doubled into both halves of a word
    h16x2 sn[8], an8[8], sq[8], aq3[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const u32 word = e < 4 ? scv.x : scv.y;
      const int sv = static_cast<int>(static_cast<int8_t>((word >> (8 * (e & 3))) & 0xFFu));
      const _Float16 sf = static_cast<_Float16>(static_cast<short>(sv));
      const _Float16 f_n = sf * static_cast<_Float16>(64.0f), a_n = sf * static_cast<_Float16>(-0.00048828125f);      // -8 * 2^-14
      const _Float16 f_q = sf * static_cast<_Float16>(128.0f), a_q = sf * static_cast<_Float16>(-0.00018310546875f);  // -3 * 2^-14
      sn[e] = h16x2{f_n, f_n};
      an8[e] = h16x2{a_n, a_n};
      sq[e] = h16x2{f_q, f_q};
      aq3[e] = h16x2{a_q, a_q};
    }
    const f32x16 zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    f32x16 acc_n = zero, acc_q = zero;
#pragma unroll
    for (int q0 = 0; q0 < 16; q0 += 4) {         // four token pages per round of operand reads, two products a page
      u32x4 a0, a1, a2, a3;
      const u32 xs = slot * kXpStageBytes;
      switch (q0) {
        case 0: lds_read128<0 * 1024>(a0, xq[0] + xs); lds_read128<1 * 1024>(a1, xq[1] + xs); lds_read128<2 * 1024>(a2, xq[2] + xs); lds_read128<3 * 1024>(a3, xq[3] + xs); break;
        case 4: lds_read128<4 * 1024>(a0, xq[4] + xs); lds_read128<5 * 1024>(a1, xq[5] + xs); lds_read128<6 * 1024>(a2, xq[6] + xs); lds_read128<7 * 1024>(a3, xq[7] + xs); break;
        case 8: lds_read128<8 * 1024>(a0, xq[8] + xs); lds_read128<9 * 1024>(a1, xq[9] + xs); lds_read128<10 * 1024>(a2, xq[10] + xs); lds_read128<11 * 1024>(a3, xq[11] + xs); break;
        default: lds_read128<12 * 1024>(a0, xq[12] + xs); lds_read128<13 * 1024>(a1, xq[13] + xs); lds_read128<14 * 1024>(a2, xq[14] + xs); lds_read128<15 * 1024>(a3, xq[15] + xs); break;
      }
      const u32x4* aq[4] = {&a0, &a1, &a2, &a3};
      u32 bn[4][4], bq[4][4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int Q = q0 + i, U = Q >> 1, H = Q & 1, hi_nib = U >> 2, gq = 2 * (U >> 2) + H;
        const int e = 2 * gq + ((U & 3) >> 1);
        const u32 t0 = ql[8 * H + 2 * (U & 3)], t1 = ql[8 * H + 2 * (U & 3) + 1];
        // nibbles to bits 4..7 of their 16-bit lanes: bytes 0 and 2, then bytes 1 and 3
        const u32 n00 = hi_nib ? t0 : t0 << 4, n01 = hi_nib ? t0 >> 8 : t0 >> 4;
        const u32 n10 = hi_nib ? t1 : t1 << 4, n11 = hi_nib ? t1 >> 8 : t1 >> 4;
        bn[i][0] = __builtin_bit_cast(u32, pk_fma_h2(n00 & 0x00F000F0u, sn[e], an8[e]));
        bn[i][1] = __builtin_bit_cast(u32, pk_fma_h2(n01 & 0x00F000F0u, sn[e], an8[e]));
        bn[i][2] = __builtin_bit_cast(u32, pk_fma_h2(n10 & 0x00F000F0u, sn[e], an8[e]));
        bn[i][3] = __builtin_bit_cast(u32, pk_fma_h2(n11 & 0x00F000F0u, sn[e], an8[e]));
        // field gq of the qh bytes to bits 4..5: shift by 4 - 2 gq (bytes 0 and 2), by -4 - 2 gq (bytes 1 and 3)
        const u32 c0 = qh[2 * (U & 3)], c1 = qh[2 * (U & 3) + 1];
        const u32 f00 = gq == 0 ? c0 << 4 : gq == 1 ? c0 << 2 : gq == 2 ? c0 : c0 >> 2, f01v = c0 >> (4 + 2 * gq);
        const u32 f10 = gq == 0 ? c1 << 4 : gq == 1 ? c1 << 2 : gq == 2 ? c1 : c1 >> 2, f11 = c1 >> (4 + 2 * gq);
        bq[i][0] = __builtin_bit_cast(u32, pk_fma_h2(f00 & 0x00300030u, sq[e], aq3[e]));
        bq[i][1] = __builtin_bit_cast(u32, pk_fma_h2(f01v & 0x00300030u, sq[e], aq3[e]));
        bq[i][2] = __builtin_bit_cast(u32, pk_fma_h2(f10 & 0x00300030u, sq[e], aq3[e]));
        bq[i][3] = __builtin_bit_cast(u32, pk_fma_h2(f11 & 0x00300030u, sq[e], aq3[e]));
      }
      lds_wait4(a0, a1, a2, a3);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const u32x4 bnv = {bn[i][0], bn[i][1], bn[i][2], bn[i][3]}, bqv = {bq[i][0], bq[i][1], bq[i][2], bq[i][3]};
        acc_n = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(h16x8, *aq[i]), __builtin_bit_cast(h16x8, bnv), acc_n, 0, 0, 0);
        acc_q = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(h16x8, *aq[i]), __builtin_bit_cast(h16x8, bqv), acc_q, 0, 0, 0);
      }
    }
    // the next tile's registers to LDS: this wave is done reading the current one
    if constexpr (NEXT) store_w();
    if constexpr (NEXT2) load_w(s + 2u);
    const float fac[8] = {__uint_as_float(f01.x), __uint_as_float(f01.y), __uint_as_float(f23.x), __uint_as_float(f23.y),
                          __uint_as_float(f45.x), __uint_as_float(f45.y), __uint_as_float(f67.x), __uint_as_float(f67.y)};
    const f32x16 other = tot;                    // the two running sums change places: each takes every other super-block
#pragma unroll
    for (int t = 0; t < 8; ++t) {
      const float fd = fac[t] * d;
#pragma unroll
      for (int pc = 0; pc < 2; ++pc) {
        const int v = 2 * t + pc;
        tot[v] = fmaf(fd, fmaf(8.0f, acc_q[v], acc_n[v]), kTwoSums ? tot_odd[v] : tot[v]);
      }
    }
    if constexpr (kTwoSums) tot_odd = other;
  };
  using std::true_type;
  using std::false_type;
  load_a(0);
  load_w(0);
  __builtin_amdgcn_sched_barrier(0);   // both sets of loads on their way before the conversion waits for the first
  convert(0);
  store_w();
  if (ns == 1u) {
    step(0u, false_type{}, false_type{});
  } else {
    load_a(1);
    load_w(1);
    u32 s = 0;
    for (; s + 2u < ns; ++s) step(s, true_type{}, true_type{});
    step(s, true_type{}, false_type{});
    step(s + 1u, false_type{}, false_type{});
  }
  const f32x16 tots[1] = {tot + tot_odd};
  finish_tiles<1>(tots, c, ws, m, n, kparts, groups, tiles, tiles, waves, group, part, tile, strip, col, g, lane, lds_flag);
}

}  // namespace gemm_f16
