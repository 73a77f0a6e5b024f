// f32 GEMV  y[n] = sum_k A[k][n] * x[k],  A is K x N row-major (trueno-gpu/src/kernels/gemv.rs: GemvKernel
// "gemv_warp_reduce" :21-166, CoalescedGemvKernel "gemv_coalesced" :188-398; both compute this product, in
// different summation orders).  Bound by HBM: 4 K N bytes of A read once.
//
// A lane owns four neighbouring columns, so a wave reads 1 KB of a row of A with one 128-bit load per lane, and
// the 8 waves of a workgroup take every eighth row of the workgroup's part of K (eight rows in flight per
// wave).  x[k] is the same for the whole wave: it comes through the scalar cache.  The waves' sums meet in LDS
// in wave order.  K is cut in parts over the grid so that the chip is filled; with several parts every part
// stores its partial y through to memory and the workgroup that arrives last at the column tile's counter adds
// the parts in part order and puts the counter back to zero - one launch, the same bits on every run.
#pragma once
#include "kquant_common.hip.h"

namespace gemv_f32 {

constexpr u32 kWaves = 8, kUnroll = 8, kTileCols = 256;

__device__ __forceinline__ void fast_body(float* __restrict__ y, const float* __restrict__ a, const float* __restrict__ x,
                                          float* __restrict__ partial, u32* __restrict__ counters, u32 k_dim, u32 n_dim,
                                          u32 rows_per_part, u32 parts) {
  __shared__ f32x4 s_sum[kWaves][64];
  __shared__ u32 s_old;
  const u32 lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
  const u32 tile = blockIdx.x / parts, part = blockIdx.x - tile * parts;
  const u32 col = tile * kTileCols + 4u * lane;
  const bool col_ok = col < n_dim;                         // n_dim % 4 == 0: a lane's four columns are all in or all out
  const u32 k0 = part * rows_per_part, k1 = min(k_dim, k0 + rows_per_part);
  const f32x4* ap = reinterpret_cast<const f32x4*>(a + (col_ok ? col : 0u));
  const size_t stride4 = n_dim >> 2;
  const __amdgpu_buffer_rsrc_t part_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      partial, 0, static_cast<int>(min(static_cast<size_t>(0x7FFFFFFF), static_cast<size_t>(parts) * n_dim * 4u)), 0x00020000);
  f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
  u32 k = k0 + wave;
  for (; k + (kUnroll - 1u) * kWaves < k1; k += kUnroll * kWaves) {
    f32x4 v[kUnroll];
    float xv[kUnroll];
#pragma unroll
    for (u32 u = 0; u < kUnroll; ++u) {
      v[u] = __builtin_nontemporal_load(ap + static_cast<size_t>(k + u * kWaves) * stride4);   // (the matrix is read once, in whole lines)
      xv[u] = x[k + u * kWaves];
    }
#pragma unroll
    for (u32 u = 0; u < kUnroll; ++u) {
      acc.x = fmaf(v[u].x, xv[u], acc.x); acc.y = fmaf(v[u].y, xv[u], acc.y);
      acc.z = fmaf(v[u].z, xv[u], acc.z); acc.w = fmaf(v[u].w, xv[u], acc.w);
    }
  }
  for (; k < k1; k += kWaves) {
    const f32x4 v = __builtin_nontemporal_load(ap + static_cast<size_t>(k) * stride4);
    const float xk = x[k];
    acc.x = fmaf(v.x, xk, acc.x); acc.y = fmaf(v.y, xk, acc.y); acc.z = fmaf(v.z, xk, acc.z); acc.w = fmaf(v.w, xk, acc.w);
  }
  s_sum[wave][lane] = acc;
  __syncthreads();
  if (wave != 0u) {
    if (parts == 1u) return;
  } else {
    for (u32 w = 1; w < kWaves; ++w) {
      const f32x4 o = s_sum[w][lane];
      acc.x += o.x; acc.y += o.y; acc.z += o.z; acc.w += o.w;
    }
    if (parts == 1u) {
      if (col_ok) *reinterpret_cast<f32x4*>(y + col) = acc;
      return;
    }
    if (col_ok)      // across workgroups (and XCDs): one 16-byte buffer store at agent scope (sc1)
      __builtin_amdgcn_raw_buffer_store_b128(u32x4{__float_as_uint(acc.x), __float_as_uint(acc.y), __float_as_uint(acc.z), __float_as_uint(acc.w)},
                                             part_rsrc, static_cast<int>((part * n_dim + col) * 4u), 0, 16);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");       // the coherent stores have been acknowledged
    if (lane == 0u) {
      const u32 old = __hip_atomic_fetch_add(counters + tile, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (old == parts - 1u) __hip_atomic_store(counters + tile, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      s_old = old;
    }
  }
  __syncthreads();
  if (wave != 0u || s_old != parts - 1u || !col_ok) return;
  float r[4] = {0.0f, 0.0f, 0.0f, 0.0f};
  for (u32 p0 = 0; p0 < parts; p0 += 16u) {                // sixteen parts in flight, added in part order
    u32x4 got[16];
#pragma unroll
    for (u32 pp = 0; pp < 16; ++pp)
      got[pp] = __builtin_amdgcn_raw_buffer_load_b128(part_rsrc, static_cast<int>((min(p0 + pp, parts - 1u) * n_dim + col) * 4u), 0, 16);
#pragma unroll
    for (u32 pp = 0; pp < 16; ++pp)
      if (p0 + pp < parts) {
        r[0] += __uint_as_float(got[pp].x); r[1] += __uint_as_float(got[pp].y);
        r[2] += __uint_as_float(got[pp].z); r[3] += __uint_as_float(got[pp].w);
      }
  }
  *reinterpret_cast<f32x4*>(y + col) = f32x4{r[0], r[1], r[2], r[3]};
}

// Any n, any alignment: a thread per column, k in order (the summation order of the reference's gemv_coalesced).
__device__ __forceinline__ void generic_body(float* __restrict__ y, const float* __restrict__ a, const float* __restrict__ x,
                                             u32 k_dim, u32 n_dim) {
  const u32 col = blockIdx.x * blockDim.x + threadIdx.x;
  if (col >= n_dim) return;
  float sum = 0.0f;
  for (u32 k = 0; k < k_dim; ++k) sum = fmaf(x[k], a[static_cast<size_t>(k) * n_dim + col], sum);
  y[col] = sum;
}

}  // namespace gemv_f32
