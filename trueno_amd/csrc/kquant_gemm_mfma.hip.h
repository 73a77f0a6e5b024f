// Batched Q4_K GEMM on the integer matrix cores (gfx950, v_mfma_i32_32x32x32_i8).
//
//   C[m x n] = A[m x k] . dequant(W[n x k])^T,  c[row*n + col]      (trueno-gpu/src/kernels/quantize.rs:568-574,
//   decode of the weights as in the GEMV family, quantize.rs:1237-1483)
//
// The quants are small integers, so the contraction runs exactly on the integer matrix cores and f32 only
// enters per (row, super-block):
//   * a first kernel turns every row of A into block fixed point: per super-block of 256 values a
//     power-of-two scale 2^(E-26) and 28-bit integers v = rint(a * 2^(26-E)), split in four 7-bit digits
//     v = d0 + 128 d1 + 128^2 d2 + 128^3 d3 (d3 signed) - four int8 "digit planes" per token, stored in the
//     matrix-core operand layout.  An element within 2^3 of its block's maximum is exact, the rest are
//     represented to 2^-27 of that maximum, i.e. better than f32 products would be;
//   * the second kernel takes 32 rows of W per wave.  Per 32-value sub-block j it builds two int8 operands
//     from the nibbles q and the 6-bit scale s_j = 8 s_hi + s_lo:  q*s_lo and q*s_hi (both <= 105), and
//     accumulates  sum q s_lo d_p  and  sum q s_hi d_p  over the whole super-block in the matrix cores'
//     int32 accumulators - no per-sub-block work outside them;
//   * per (row, token, plane, super-block):  acc += 2^(E-26) 128^p * d * (S_lo + 8 S_hi), and per (row, token,
//     super-block) the min term  dmin * sum_j m_j * (sum of a over sub-block j)  in f32, as the GEMV has it.
//
// Operand layout (A operand = digit planes, 32 rows = 8 tokens x 4 planes, row = 4*token + plane;
// B operand = 32 rows of W): lane l supplies A[row l%32][k = 16*(l/32) .. +15] and B[k = 16*(l/32) .. +15][col l%32];
// D[row 8*(v/4) + 4*(l/32) + v%4][col l%32] arrives in lane l, register v.  So lane l ends up with, for W row
// l%32, the tokens 2*(v/4) + l/32 and the planes v%4.
#pragma once
#include "kquant_common.hip.h"

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));

namespace gemm_mfma {

constexpr u32 kTokensPerTile = 8;
constexpr u32 kTileSbBytes = 8 * 1024;    // digit planes of one token tile for one super-block: 8 sub-blocks x 1 KB
constexpr u32 kMetaSbFloats = 72;         // per token tile and super-block: 8 block scales [token], 64 sub-block sums [token][j]

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

// Pre-pass.  One wave per (token, super-block) of the padded token range [0, 8*tiles); tokens >= m give zero
// planes.  Also clears C (the main kernel may add two partial results into it).
//   planes: ((tile*nsb + sb)*8 + j)*1024 + kc*512 + (4*(token%8) + p)*16 + b  = digit p of value 32j + 16kc + b
//   meta  : (tile*nsb + sb)*72 + token%8                 f32 = 2^(E-26), the weight of digit plane 0
//           (tile*nsb + sb)*72 + 8 + (token%8)*8 + j     f32 = sum of a over sub-block j
__device__ __forceinline__ void planes_body(const float* __restrict__ a, uint8_t* __restrict__ planes, float* __restrict__ meta,
                                            float* __restrict__ c, u32 m, u32 n, u32 k, u32 clear_c) {
  const u32 lane = threadIdx.x & 63u, wave = threadIdx.x >> 6, waves = blockDim.x >> 6;
  const u32 nsb = k >> 8, tiles = (m + kTokensPerTile - 1) / kTokensPerTile;
  const u32 items = tiles * kTokensPerTile * nsb;
  for (u32 it = blockIdx.x * waves + wave; it < items; it += gridDim.x * waves) {
    const u32 token = it / nsb, sb = it - token * nsb;
    const u32 tile = token >> 3, tl = token & 7u;
    f32x4 v = {0.0f, 0.0f, 0.0f, 0.0f};
    if (token < m) v = reinterpret_cast<const f32x4*>(a + static_cast<size_t>(token) * k + 256u * sb)[lane];
    const u32 a0 = __float_as_uint(v.x) & 0x7FFFFFFFu, a1 = __float_as_uint(v.y) & 0x7FFFFFFFu;
    const u32 a2 = __float_as_uint(v.z) & 0x7FFFFFFFu, a3 = __float_as_uint(v.w) & 0x7FFFFFFFu;
    const u32 amax = wave_max_u32(max(max(a0, a1), max(a2, a3)));
    u32 e = amax >> 23;                       // biased exponent of the block maximum
    const bool finite = e != 255u;
    e = e < 27u ? 27u : e;                    // keeps both scales normal; a tiny block loses nothing that matters
    const float scale = __uint_as_float((280u - e) << 23);   // 2^(26 - E)
    const float xs[4] = {v.x, v.y, v.z, v.w};
    u32 plane[4] = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int iv = finite ? __float2int_rn(xs[q] * scale) : 0;     // |iv| <= 2^27
      plane[0] |= (static_cast<u32>(iv) & 127u) << (8 * q);
      plane[1] |= ((static_cast<u32>(iv) >> 7) & 127u) << (8 * q);
      plane[2] |= ((static_cast<u32>(iv) >> 14) & 127u) << (8 * q);
      plane[3] |= (static_cast<u32>(iv >> 21) & 255u) << (8 * q);
    }
    const u32 j = lane >> 3, kc = (lane >> 2) & 1u, b = (lane & 3u) * 4u;
    uint8_t* dst = planes + (static_cast<size_t>(tile) * nsb + sb) * kTileSbBytes + j * 1024u + kc * 512u + (4u * tl) * 16u + b;
#pragma unroll
    for (int p = 0; p < 4; ++p) *reinterpret_cast<u32*>(dst + 16 * p) = plane[p];
    float* mt = meta + (static_cast<size_t>(tile) * nsb + sb) * kMetaSbFloats;
    // a block holding an infinity or a NaN poisons its outputs, as the f32 product would
    if (lane == 0u) mt[tl] = finite ? __uint_as_float((e - 26u) << 23) : __uint_as_float(0x7FC00000u);
    float sj = (v.x + v.y) + (v.z + v.w);
    sj += dpp_f32<0xB1>(sj);
    sj += dpp_f32<0x4E>(sj);
    sj += dpp_f32<0x141>(sj);                 // all 8 lanes of a sub-block hold its sum
    if ((lane & 7u) == 0u) mt[8u + tl * 8u + j] = sj;
  }
  if (clear_c) {
    const size_t total = static_cast<size_t>(m) * n;
    for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < total; i += static_cast<size_t>(gridDim.x) * blockDim.x)
      c[i] = 0.0f;
  }
}

__device__ __forceinline__ u32 pk_mul_u16(u32 a, u32 b) {
  const u16x2 r = __builtin_bit_cast(u16x2, a) * __builtin_bit_cast(u16x2, b);
  return __builtin_bit_cast(u32, r);
}

// Main kernel: one workgroup = 32 rows of W (blockIdx.x) x T token tiles (blockIdx.y) x one part of K (blockIdx.z
// of gridDim.z parts); its waves cut that part of K in equal runs of super-blocks and meet in LDS, where wave 0
// adds their results in wave order.  With gridDim.z == 1 the result is stored; otherwise it is added to C, which
// the pre-pass cleared (two parts at most, so the sum does not depend on which part arrives first).
//   static LDS = waves(<= 4) * T * 4 * 64 floats
template <int T>
__device__ __forceinline__ void q4k_body(const uint8_t* __restrict__ planes, const float* __restrict__ meta,
                                         const uint8_t* __restrict__ w, float* __restrict__ c, u32 m, u32 n, u32 k) {
  __shared__ float s_part[4][T * 4][64];
  const u32 lane = threadIdx.x & 63u, wave = threadIdx.x >> 6, waves = min(blockDim.x >> 6, 4u);
  const u32 nsb = k >> 8, tiles = (m + kTokensPerTile - 1) / kTokensPerTile;
  const u32 col = lane & 31u, kc = lane >> 5;
  u32 row = blockIdx.x * 32u + col;
  const bool row_ok = row < n;
  row = row_ok ? row : n - 1u;
  const u32 tile0 = blockIdx.y * T;
  const u32 part_begin = static_cast<u32>((static_cast<uint64_t>(nsb) * blockIdx.z) / gridDim.z);
  const u32 part_end = static_cast<u32>((static_cast<uint64_t>(nsb) * (blockIdx.z + 1)) / gridDim.z);
  const u32 wv = min(wave, waves - 1u);
  const u32 sb_begin = part_begin + ((part_end - part_begin) * wv) / waves;
  const u32 sb_end = wave < waves ? part_begin + ((part_end - part_begin) * (wv + 1u)) / waves : sb_begin;
  const uint8_t* rp = w + static_cast<size_t>(row) * nsb * 144u;
  const uint8_t* ap[T];
  const float* mp[T];
#pragma unroll
  for (int t = 0; t < T; ++t) {
    const u32 tile = min(tile0 + t, tiles - 1u);
    ap[t] = planes + static_cast<size_t>(tile) * nsb * kTileSbBytes + kc * 512u + col * 16u;
    mp[t] = meta + static_cast<size_t>(tile) * nsb * kMetaSbFloats;
  }

  float acc[T][16], accm[T][4];
#pragma unroll
  for (int t = 0; t < T; ++t) {
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[t][v] = 0.0f;
#pragma unroll
    for (int g = 0; g < 4; ++g) accm[t][g] = 0.0f;
  }

  // operands of the next super-block are loaded while the current one is multiplied
  u32x4 hdr, q[4];
  v4i an[T][8];
  float pwn[T][4];
  f32x4 sxn[T][8];
  auto load_sb = [&](u32 sb) {
    const uint8_t* bp = rp + static_cast<size_t>(sb) * 144u;
    hdr = load128(bp);
#pragma unroll
    for (int cc = 0; cc < 4; ++cc) q[cc] = load128(bp + 16 + 32 * cc + 16 * kc);
#pragma unroll
    for (int t = 0; t < T; ++t)
#pragma unroll
      for (int j = 0; j < 8; ++j)
        an[t][j] = *reinterpret_cast<const v4i*>(ap[t] + static_cast<size_t>(sb) * kTileSbBytes + j * 1024u);
#pragma unroll
    for (int t = 0; t < T; ++t) {
      const float* mf = mp[t] + static_cast<size_t>(sb) * kMetaSbFloats;
      const f32x4* mt = reinterpret_cast<const f32x4*>(mf);
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        pwn[t][g] = mf[2u * g + kc];                      // block scale of token 2g + kc
        sxn[t][2 * g] = mt[2u + (2u * g + kc) * 2u];      // its eight sub-block sums
        sxn[t][2 * g + 1] = mt[2u + (2u * g + kc) * 2u + 1u];
      }
    }
  };
  if (sb_begin < sb_end) load_sb(sb_begin);
  for (u32 sb = sb_begin; sb < sb_end; ++sb) {
    const u32x4 h = hdr;
    u32x4 qq[4];
    v4i a[T][8];
#pragma unroll
    for (int cc = 0; cc < 4; ++cc) qq[cc] = q[cc];
#pragma unroll
    for (int t = 0; t < T; ++t)
#pragma unroll
      for (int j = 0; j < 8; ++j) a[t][j] = an[t][j];
    const float d = half_bits_to_f32(h.x), dmin = half_bits_to_f32(h.x >> 16);
    // eight 6-bit scales and mins as bytes (get_scale_min_k4, quantize.rs:1306-1385)
    const u32 s_lo4 = h.y & 0x3F3F3F3Fu, m_lo4 = h.z & 0x3F3F3F3Fu;
    const u32 s_hi4 = (h.w & 0x0F0F0F0Fu) | ((h.y >> 2) & 0x30303030u);
    const u32 m_hi4 = ((h.w >> 4) & 0x0F0F0F0Fu) | ((h.z >> 2) & 0x30303030u);
    // the min term first: its operands are then dead before the next super-block's loads are issued
    const float mn[8] = {ubyte0(m_lo4), ubyte1(m_lo4), ubyte2(m_lo4), ubyte3(m_lo4),
                         ubyte0(m_hi4), ubyte1(m_hi4), ubyte2(m_hi4), ubyte3(m_hi4)};
    float pwc[T][4];
#pragma unroll
    for (int t = 0; t < T; ++t) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        pwc[t][g] = pwn[t][g];
        const f32x4 s0 = sxn[t][2 * g], s1 = sxn[t][2 * g + 1];
        float ms = mn[0] * s0.x;
        ms = fmaf(mn[1], s0.y, ms); ms = fmaf(mn[2], s0.z, ms); ms = fmaf(mn[3], s0.w, ms);
        ms = fmaf(mn[4], s1.x, ms); ms = fmaf(mn[5], s1.y, ms); ms = fmaf(mn[6], s1.z, ms); ms = fmaf(mn[7], s1.w, ms);
        accm[t][g] = fmaf(dmin, ms, accm[t][g]);
      }
    }
    if (sb + 1 < sb_end) load_sb(sb + 1);
    v16i dlo[T], dhi[T];
#pragma unroll
    for (int t = 0; t < T; ++t) {
      dlo[t] = v16i{0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
      dhi[t] = dlo[t];
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const u32 s = ((j < 4 ? s_lo4 : s_hi4) >> (8 * (j & 3))) & 0xFFu;
      const u32 slo = (s & 7u) * 0x00010001u, shi = (s >> 3) * 0x00010001u;
      v4i blo, bhi;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const u32 nib = (qq[j >> 1][i] >> (4 * (j & 1))) & 0x0F0F0F0Fu;
        blo[i] = static_cast<int>(pk_mul_u16(nib, slo));
        bhi[i] = static_cast<int>(pk_mul_u16(nib, shi));
      }
#pragma unroll
      for (int t = 0; t < T; ++t) {
        dlo[t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[t][j], blo, dlo[t], 0, 0, 0);
        dhi[t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[t][j], bhi, dhi[t], 0, 0, 0);
      }
    }
#pragma unroll
    for (int t = 0; t < T; ++t) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const float w0 = pwc[t][g] * d;                        // exact powers of two times d
        const float pws[4] = {w0, w0 * 128.0f, w0 * 16384.0f, w0 * 2097152.0f};
#pragma unroll
        for (int p = 0; p < 4; ++p) {
          const int v = 4 * g + p;
          const float sq = static_cast<float>(dlo[t][v] + 8 * dhi[t][v]);
          acc[t][v] = fmaf(pws[p], sq, acc[t][v]);
        }
      }
    }
  }
#pragma unroll
  for (int t = 0; t < T; ++t)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const float r = (acc[t][4 * g] + acc[t][4 * g + 1]) + (acc[t][4 * g + 2] + acc[t][4 * g + 3]);
      if (wave < waves) s_part[wave][t * 4 + g][lane] = r - accm[t][g];
    }
  __syncthreads();
  if (wave != 0u || !row_ok) return;
  const u32 out_row = blockIdx.x * 32u + col;
#pragma unroll
  for (int t = 0; t < T; ++t) {
    if (tile0 + t >= tiles) break;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const u32 token = (tile0 + t) * kTokensPerTile + 2u * g + kc;
      if (token < m) {
        float r = s_part[0][t * 4 + g][lane];
        for (u32 i = 1; i < waves; ++i) r += s_part[i][t * 4 + g][lane];
        float* dst = c + static_cast<size_t>(token) * n + out_row;
        if (gridDim.z == 1) *dst = r;
        else atomicAdd(dst, r);
      }
    }
  }
}

}  // namespace gemm_mfma
