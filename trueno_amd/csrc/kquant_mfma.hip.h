// Integer matrix-core form of the k-quant dot products (gfx950, v_mfma_i32_32x32x32_i8).
//
// Idea.  The VALU form spends ~3 lane-operations per weight (convert + FMA + unpack) and is
// issue-bound well below the HBM roofline.  Here the multiply-accumulate moves to the matrix
// cores and stays exact:
//   * the weights go in as they are stored - masked 4-bit quants as int8 (B operand), no
//     conversion to floating point at all;
//   * the activations are converted once per workgroup to block fixed point: per super-block of
//     256 values a power-of-two scale 2^(E-26) and a 28-bit signed integer v = rint(x * 2^(26-E)),
//     split in four 7-bit digits v = d0 + 128 d1 + 128^2 d2 + 128^3 d3 (d3 signed): four int8
//     "digit planes" (A operand rows).  Every element within 2^3 of the block maximum is
//     represented exactly; the rest to 2^-27 of the block maximum;
//   * one MFMA gives, for 32 matrix rows at once, the exact integer sums  sum_k q[n,k] d_p[k]
//     over one 32-value sub-block for all planes p; the 6-bit sub-block scale is applied by an
//     integer multiply-add, so a whole super-block accumulates in exact integer arithmetic;
//   * per (row, super-block) there are then a handful of f32 operations: the four planes are
//     recombined with their power-of-two weights, multiplied by d, and the min term
//     dmin * sum_j m_j * sum_{k in j} x_k is subtracted.
// f32 rounding happens only in those last steps and in the sum over super-blocks, so the result
// is closer to the fp64 product than an f32 FMA chain over k.
//
// Lane roles in a tile of 32 rows x 1 super-block: lane l holds row r = l % 32 and k-half
// kc = l / 32 (the 16 values 16kc..16kc+15 of every sub-block).  A-operand row i is fed by lanes
// with l % 32 == i; rows 0,1,4,5 carry planes 0,1,2,3 and every other row carries a copy of some
// plane (its results are never read).  D row 8(v/4) + 4(l/32) + v%4 lands in lane l, register v,
// so lanes 0..31 read planes 0,1 and lanes 32..63 read planes 2,3 from registers 0,1.
//
// Decode followed: trueno-gpu/src/kernels/quantize.rs:1237-1483 (Q4_K).
#pragma once
#include "kquant_common.hip.h"

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

namespace mfma {

constexpr u32 kPlaneBytesPerSb = 1024;                 // 8 sub-blocks x 2 k-halves x 4 planes x 16 B
constexpr u32 kMetaBytesPerSb = 64;                    // 4 plane weights, 8 sub-block sums, pad
constexpr u32 kLdsBytesPerSb = kPlaneBytesPerSb + kMetaBytesPerSb;

template <int CTRL>
__device__ __forceinline__ u32 dpp_u32(u32 v) {
  return static_cast<u32>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), CTRL, 0xF, 0xF, true));
}

__device__ __forceinline__ u32 wave_max_u32(u32 v) {
  v = max(v, dpp_u32<0xB1>(v));
  v = max(v, dpp_u32<0x4E>(v));
  v = max(v, dpp_u32<0x141>(v));
  v = max(v, dpp_u32<0x140>(v));
  const u32 a = static_cast<u32>(__builtin_amdgcn_readlane(static_cast<int>(v), 0));
  const u32 b = static_cast<u32>(__builtin_amdgcn_readlane(static_cast<int>(v), 16));
  const u32 c = static_cast<u32>(__builtin_amdgcn_readlane(static_cast<int>(v), 32));
  const u32 d = static_cast<u32>(__builtin_amdgcn_readlane(static_cast<int>(v), 48));
  return max(max(a, b), max(c, d));
}

// One wave converts one super-block of activations (256 f32 at xsb) into its LDS image at `dst`:
//   planes: byte [j*128 + kc*64 + p*16 + b] = digit p of value 32j + 16kc + b
//   meta  : f32 [0..3] plane weights 2^(E-26) * 128^p, f32 [4..11] sum of x over sub-block j
// A block holding an infinity or a NaN gets NaN plane weights (the output row becomes NaN).
__device__ __forceinline__ void convert_superblock(const float* __restrict__ xsb, uint8_t* __restrict__ dst, u32 lane) {
  const f32x4 v = reinterpret_cast<const f32x4*>(xsb)[lane];
  const u32 a0 = __float_as_uint(v.x) & 0x7FFFFFFFu, a1 = __float_as_uint(v.y) & 0x7FFFFFFFu;
  const u32 a2 = __float_as_uint(v.z) & 0x7FFFFFFFu, a3 = __float_as_uint(v.w) & 0x7FFFFFFFu;
  const u32 amax = wave_max_u32(max(max(a0, a1), max(a2, a3)));
  u32 e = amax >> 23;                       // biased exponent of the block maximum
  const bool finite = e != 255u;
  e = e < 27u ? 27u : e;                    // keeps both scales normal; tiny blocks lose nothing that matters
  const float scale = __uint_as_float((280u - e) << 23);   // 2^(26 - E)
  const float xs[4] = {v.x, v.y, v.z, v.w};
  u32 plane[4] = {0u, 0u, 0u, 0u};
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const int iv = __float2int_rn(xs[q] * scale);          // |iv| <= 2^27
    plane[0] |= (static_cast<u32>(iv) & 127u) << (8 * q);
    plane[1] |= ((static_cast<u32>(iv) >> 7) & 127u) << (8 * q);
    plane[2] |= ((static_cast<u32>(iv) >> 14) & 127u) << (8 * q);
    plane[3] |= (static_cast<u32>(iv >> 21) & 255u) << (8 * q);
  }
  const u32 j = lane >> 3, kc = (lane >> 2) & 1u;
  u32* p32 = reinterpret_cast<u32*>(dst + j * 128u + kc * 64u + (lane & 3u) * 4u);
  p32[0] = plane[0];
  p32[4] = plane[1];
  p32[8] = plane[2];
  p32[12] = plane[3];
  float s = (v.x + v.y) + (v.z + v.w);
  s += dpp_f32<0xB1>(s);
  s += dpp_f32<0x4E>(s);
  s += dpp_f32<0x141>(s);                   // all 8 lanes of a sub-block hold its sum
  float* meta = reinterpret_cast<float*>(dst + kPlaneBytesPerSb);
  if ((lane & 7u) == 0u) meta[4 + j] = s;
  if (lane < 4u) {
    const float pw = __uint_as_float((e - 26u + 7u * lane) << 23);   // 2^(E-26) * 128^lane
    meta[lane] = finite ? pw : __uint_as_float(0x7FC00000u);
  }
}

// Q4_K tile: 32 rows x 1 super-block.
struct Q4Tile {
  u32x4 hdr, q[4];
};

__device__ __forceinline__ void q4k_tile_load(Q4Tile& t, const uint8_t* __restrict__ sbp, u32 kc) {
  t.hdr = load128(sbp);
#pragma unroll
  for (int c = 0; c < 4; ++c) t.q[c] = load128(sbp + 16 + 32 * c + 16 * kc);
}

// sum over the super-block of w*x for row (lane % 32): this lane's half of it - lanes < 32 carry
// planes 0,1 and sub-blocks 0..3 of the min term, lanes >= 32 planes 2,3 and sub-blocks 4..7; the
// caller adds the two halves.
__device__ __forceinline__ float q4k_tile_dot(const Q4Tile& t, const uint8_t* __restrict__ lds_sb, u32 lane) {
  const u32 half = lane >> 5, r = lane & 31u;
  const float d = half_bits_to_f32(t.hdr.x);
  const float dmin = half_bits_to_f32(t.hdr.x >> 16);
  // eight 6-bit scales and mins as bytes (get_scale_min_k4, quantize.rs:1306-1385)
  const u32 s_lo = t.hdr.y & 0x3F3F3F3Fu, m_lo = t.hdr.z & 0x3F3F3F3Fu;
  const u32 s_hi = (t.hdr.w & 0x0F0F0F0Fu) | ((t.hdr.y >> 2) & 0x30303030u);
  const u32 m_hi = ((t.hdr.w >> 4) & 0x0F0F0F0Fu) | ((t.hdr.z >> 2) & 0x30303030u);
  const u32 arow = ((r & 1u) | ((r >> 1) & 2u)) * 16u + half * 64u;   // plane carried by A row r, this k-half
  const v16i zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
  int acc0 = 0, acc1 = 0;
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    const u32x4 qv = t.q[c];
    v4i blo, bhi;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      blo[i] = static_cast<int>(qv[i] & 0x0F0F0F0Fu);
      bhi[i] = static_cast<int>((qv[i] >> 4) & 0x0F0F0F0Fu);
    }
    const v4i alo = *reinterpret_cast<const v4i*>(lds_sb + (2 * c) * 128 + arow);
    const v4i ahi = *reinterpret_cast<const v4i*>(lds_sb + (2 * c + 1) * 128 + arow);
    const v16i dlo = __builtin_amdgcn_mfma_i32_32x32x32_i8(alo, blo, zero, 0, 0, 0);
    const v16i dhi = __builtin_amdgcn_mfma_i32_32x32x32_i8(ahi, bhi, zero, 0, 0, 0);
    const u32 sp = c < 2 ? s_lo : s_hi;
    const int sc0 = static_cast<int>((sp >> (16 * (c & 1))) & 0xFFu);
    const int sc1 = static_cast<int>((sp >> (16 * (c & 1) + 8)) & 0xFFu);
    acc0 = __mul24(dlo[0], sc0) + acc0;
    acc1 = __mul24(dlo[1], sc0) + acc1;
    acc0 = __mul24(dhi[0], sc1) + acc0;
    acc1 = __mul24(dhi[1], sc1) + acc1;
  }
  const float* meta = reinterpret_cast<const float*>(lds_sb + kPlaneBytesPerSb);
  const f32x2 pw = *reinterpret_cast<const f32x2*>(meta + 2 * half);
  const f32x4 sx = *reinterpret_cast<const f32x4*>(meta + 4 + 4 * half);
  const float f = fmaf(pw.y, static_cast<float>(acc1), pw.x * static_cast<float>(acc0));
  const u32 mp = half ? m_hi : m_lo;
  float mins = ubyte0(mp) * sx.x;
  mins = fmaf(ubyte1(mp), sx.y, mins);
  mins = fmaf(ubyte2(mp), sx.z, mins);
  mins = fmaf(ubyte3(mp), sx.w, mins);
  return fmaf(d, f, -(dmin * mins));
}

// y[n] = sum_k W[n,k] x[k], Q4_K.  Workgroup = W waves sharing a run of 32-row tiles; wave w takes
// super-blocks w, w+W, ... of every tile; partial sums meet in LDS.
//   dynamic LDS = nsb * kLdsBytesPerSb + tiles_per_block * W * 128 bytes
__device__ __forceinline__ void q4k_gemv_mfma_body(float* __restrict__ y, const uint8_t* __restrict__ w,
                                                   const float* __restrict__ x, u32 k_dim, u32 n_dim) {
  extern __shared__ f32x4 lds4[];
  uint8_t* lds = reinterpret_cast<uint8_t*>(lds4);
  const u32 tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6, waves = blockDim.x >> 6;
  const u32 nsb = k_dim >> 8;
  if (waves == 0 || nsb == 0 || n_dim == 0) return;
  const u32 tiles = (n_dim + 31u) >> 5;
  const u32 tiles_per_block = (tiles + gridDim.x - 1) / gridDim.x;
  const u32 tile0 = blockIdx.x * tiles_per_block;
  if (tile0 >= tiles) return;
  const u32 my_tiles = min(tiles_per_block, tiles - tile0);
  const u32 my_nsb = wave < nsb ? (nsb - wave + waves - 1) / waves : 0u;
  const u32 n_it = my_tiles * my_nsb;
  const u32 r = lane & 31u, kc = lane >> 5;
  const size_t row_bytes = static_cast<size_t>(nsb) * 144u;

  auto issue = [&](Q4Tile& t, u32 it) {
    const u32 tl = it / my_nsb, sb = wave + (it - tl * my_nsb) * waves;
    u32 row = (tile0 + tl) * 32u + r;
    row = row < n_dim ? row : n_dim - 1;
    q4k_tile_load(t, w + row * row_bytes + static_cast<size_t>(sb) * 144u, kc);
  };
  Q4Tile ta, tb;
  if (n_it > 0) issue(ta, 0);               // weights are in flight while the activations are converted

  for (u32 sb = wave; sb < nsb; sb += waves) convert_superblock(x + 256u * sb, lds + sb * kLdsBytesPerSb, lane);
  float* part = reinterpret_cast<float*>(lds + nsb * kLdsBytesPerSb);
  __syncthreads();

  float row_acc = 0.0f;
  auto consume = [&](const Q4Tile& t, u32 it) {
    const u32 tl = it / my_nsb, si = it - tl * my_nsb, sb = wave + si * waves;
    row_acc += q4k_tile_dot(t, lds + sb * kLdsBytesPerSb, lane);
    if (si == my_nsb - 1) {
      const float other = __shfl_xor(row_acc, 32);
      if (lane < 32u) part[(tl * waves + wave) * 32u + lane] = row_acc + other;
      row_acc = 0.0f;
    }
  };
  u32 it = 0;
  for (; it + 2 <= n_it; it += 2) {
    issue(tb, it + 1);
    consume(ta, it);
    if (it + 2 < n_it) issue(ta, it + 2);
    consume(tb, it + 1);
  }
  if (it < n_it) consume(ta, it);
  __syncthreads();
  const u32 contributors = waves < nsb ? waves : nsb;
  for (u32 t = tid; t < my_tiles * 32u; t += blockDim.x) {
    const u32 tl = t >> 5, rr = t & 31u, row = (tile0 + tl) * 32u + rr;
    if (row < n_dim) {
      float s = part[(tl * waves) * 32u + rr];
      for (u32 i = 1; i < contributors; ++i) s += part[(tl * waves + i) * 32u + rr];
      y[row] = s;
    }
  }
}


// ------------------------------------------------------------------------------------------
// Staged form.  Reading the B operand straight from global memory makes every wave-load touch 32
// rows (adjacent lanes 2304+ bytes apart), which the memory pipeline serves at barely half the
// rate of a contiguous stream.  Here a wave streams its sub-tile - 32 rows x S super-blocks, i.e.
// 32 contiguous runs of S*144 bytes - with adjacent lanes on adjacent 16-byte pieces, parks it in
// a wave-private LDS area whose row stride (S*144 + 16) spreads 16 consecutive rows over all
// banks, and reads it back in operand layout.  The area belongs to one wave, so the main loop
// has no barrier: LDS operations of a wave execute in order.
//   dynamic LDS = nsb*kLdsBytesPerSb + tiles_per_block*W*128 + W*32*(S*144+16)
// Needs n_dim >= 32 (a ragged last tile is shifted back to rows n-32..n-1 and recomputes a few
// rows with identical results).
// ------------------------------------------------------------------------------------------
template <int S>
__device__ __forceinline__ void q4k_gemv_mfma_staged_body(float* __restrict__ y, const uint8_t* __restrict__ w,
                                                          const float* __restrict__ x, u32 k_dim, u32 n_dim) {
  constexpr u32 kSeg = S * 144u, kRowStride = kSeg + 16u, kStage = 32u * kRowStride;
  constexpr u32 kPiecesPerRow = S * 9u;                         // 16-byte pieces in one row segment
  constexpr u32 kLoads = (32u * kPiecesPerRow + 63u) / 64u;     // wave-loads per sub-tile
  extern __shared__ f32x4 lds4[];
  uint8_t* lds = reinterpret_cast<uint8_t*>(lds4);
  const u32 tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6, waves = blockDim.x >> 6;
  const u32 nsb = k_dim >> 8;
  if (waves == 0 || nsb == 0 || n_dim < 32u) return;
  const u32 tiles = (n_dim + 31u) >> 5;
  const u32 tiles_per_block = (tiles + gridDim.x - 1) / gridDim.x;
  const u32 tile0 = blockIdx.x * tiles_per_block;
  if (tile0 >= tiles) return;
  const u32 my_tiles = min(tiles_per_block, tiles - tile0);
  const u32 groups = (nsb + S - 1) / S;                         // sub-tiles (groups of S super-blocks) per tile
  const u32 my_groups = wave < groups ? (groups - wave + waves - 1) / waves : 0u;
  const u32 n_it = my_tiles * my_groups;
  const size_t row_bytes = static_cast<size_t>(nsb) * 144u;

  // per-lane piece geometry (does not depend on the sub-tile)
  u32 g_off[kLoads], l_off[kLoads];
#pragma unroll
  for (u32 i = 0; i < kLoads; ++i) {
    u32 p = lane + 64u * i;
    p = p < 32u * kPiecesPerRow ? p : 32u * kPiecesPerRow - 1;  // tail lanes repeat the last piece
    const u32 row = p / kPiecesPerRow, col = p - row * kPiecesPerRow;
    g_off[i] = row * static_cast<u32>(row_bytes) + col * 16u;
    l_off[i] = row * kRowStride + col * 16u;
  }
  auto tile_row0 = [&](u32 tl) {
    const u32 r0 = (tile0 + tl) * 32u;
    return r0 + 32u <= n_dim ? r0 : n_dim - 32u;
  };
  // a ragged last group (fewer than S super-blocks left) is shifted back too
  auto group_sb0 = [&](u32 gi) {
    const u32 sb0 = (wave + gi * waves) * S;
    return sb0 + S <= nsb ? sb0 : nsb - S;
  };
  u32x4 stage_regs[kLoads];
  auto issue = [&](u32 it) {
    const u32 tl = it / my_groups, gi = it - tl * my_groups;
    const uint8_t* base = w + tile_row0(tl) * row_bytes + static_cast<size_t>(group_sb0(gi)) * 144u;
#pragma unroll
    for (u32 i = 0; i < kLoads; ++i) stage_regs[i] = load128(base + g_off[i]);
  };
  if (n_it > 0) issue(0);

  for (u32 sb = wave; sb < nsb; sb += waves) convert_superblock(x + 256u * sb, lds + sb * kLdsBytesPerSb, lane);
  float* part = reinterpret_cast<float*>(lds + nsb * kLdsBytesPerSb);
  uint8_t* stage = lds + nsb * kLdsBytesPerSb + tiles_per_block * waves * 128u + wave * kStage;
  __syncthreads();

  const u32 r = lane & 31u, kc = lane >> 5;
  float row_acc = 0.0f;
  for (u32 it = 0; it < n_it; ++it) {
    const u32 tl = it / my_groups, gi = it - tl * my_groups;
#pragma unroll
    for (u32 i = 0; i < kLoads; ++i) *reinterpret_cast<u32x4*>(stage + l_off[i]) = stage_regs[i];
    if (it + 1 < n_it) issue(it + 1);
    const u32 sb0 = group_sb0(gi);
    const u32 first = (wave + gi * waves) * S;                  // super-blocks below `first` belong to another group
#pragma unroll
    for (u32 s = 0; s < static_cast<u32>(S); ++s) {
      const uint8_t* sbp = stage + r * kRowStride + s * 144u;
      Q4Tile t;
      t.hdr = *reinterpret_cast<const u32x4*>(sbp);
#pragma unroll
      for (int c = 0; c < 4; ++c) t.q[c] = *reinterpret_cast<const u32x4*>(sbp + 16 + 32 * c + 16 * kc);
      const float v = q4k_tile_dot(t, lds + (sb0 + s) * kLdsBytesPerSb, lane);
      row_acc += (sb0 + s >= first) ? v : 0.0f;
    }
    if (gi == my_groups - 1) {
      const float other = __shfl_xor(row_acc, 32);
      if (lane < 32u) part[(tl * waves + wave) * 32u + lane] = row_acc + other;
      row_acc = 0.0f;
    }
  }
  __syncthreads();
  const u32 contributors = waves < groups ? waves : groups;
  for (u32 t = tid; t < my_tiles * 32u; t += blockDim.x) {
    const u32 tl = t >> 5, rr = t & 31u, row = tile_row0(tl) + rr;
    float s = part[(tl * waves) * 32u + rr];
    for (u32 i = 1; i < contributors; ++i) s += part[(tl * waves + i) * 32u + rr];
    y[row] = s;
  }
}

}  // namespace mfma
