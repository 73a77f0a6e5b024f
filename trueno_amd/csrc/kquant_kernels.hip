// gfx950 kernels for the fused k-quant matrix path: dequantise-and-multiply GEMV (Q4_K, Q5_K,
// Q6_K), the batched quantized GEMM and the dequantise-to-f32 test surface.
//
// Exported kernel names and parameter lists are the reference's
// (trueno-gpu/src/kernels/quantize.rs): q4k_gemv_warp_reduce :1183-1194, q5k_gemv_warp_reduce
// :1548-1558, q6k_gemv_warp_reduce :1749-1775, q4k_gemm_ggml :353-359, q5k_gemm_ggml :644-650,
// q6k_gemm_ggml :930-936.  Launch geometry differs from the reference's (grid = N blocks of one
// 32-thread warp, :1151-1155): here it is a property of the kernel, chosen by the host library,
// and every kernel gives the same result for any grid size and any block size that is a
// multiple of 64.
#include "kquant_quarter.hip.h"

// ------------------------------------------------------------------------------------------
// Fast GEMV body.  One workgroup owns R consecutive rows; the activation vector is staged once
// into LDS (swizzled), then each wave keeps its 64-activations-per-lane slice in registers and
// streams rows: U rows of loads in flight per wave, unpack in registers, factorised dot, wave
// reduction.  K is cut in slabs of 16 super-blocks (one wave-width); with S slabs, min(S, waves)
// waves share a row and their partial sums meet in LDS.
//   dynamic LDS = K*4 bytes (activations) + Sw*R*4 bytes (partial sums)
// ------------------------------------------------------------------------------------------
template <int FMT, int U>
__device__ __forceinline__ void gemv_fast_body(float* __restrict__ y, const uint8_t* __restrict__ w,
                                               const float* __restrict__ x, u32 k_dim, u32 n_dim,
                                               u32 block_id, u32 num_blocks) {
  using Q = Quarter<FMT>;
  extern __shared__ f32x4 lds4[];
  const u32 tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6, waves = blockDim.x >> 6;
  const u32 nsb = k_dim >> 8;
  if (waves == 0 || nsb == 0 || n_dim == 0) return;
  const u32 slabs = (nsb + 15u) >> 4;
  const u32 sw_count = slabs < waves ? slabs : waves;  // waves sharing one row
  const u32 groups = waves / sw_count;                 // row groups per workgroup
  const u32 ug = U * groups;
  u32 rows_per_block = (n_dim + num_blocks - 1) / num_blocks;
  rows_per_block = ((rows_per_block + ug - 1) / ug) * ug;
  const u32 row0 = block_id * rows_per_block;
  if (row0 >= n_dim) return;

  const u32 units = k_dim >> 2;
  const f32x4* x4 = reinterpret_cast<const f32x4*>(x);
  for (u32 u = tid; u < units; u += blockDim.x) lds4[Q::swz(u)] = x4[u];
  float* part = reinterpret_cast<float*>(lds4 + units);
  __syncthreads();

  const u32 sw = wave % sw_count, grp = wave / sw_count;
  if (grp < groups) {
    const u32 sbl = lane >> 2, c = lane & 3u;
    const size_t row_bytes = static_cast<size_t>(nsb) * Q::SB;
    const u32 batches = rows_per_block / ug;
    for (u32 slab = sw; slab < slabs; slab += sw_count) {
      const u32 sb = slab * 16u + sbl;
      const bool valid = sb < nsb;
      const u32 sbc = valid ? sb : nsb - 1;
      float xr[64];
      float sx[Q::NSUM];
#pragma unroll
      for (int s = 0; s < Q::NSUM; ++s) sx[s] = 0.0f;
#pragma unroll
      for (int q = 0; q < 16; ++q) {
        const u32 unit = (256u * sbc + Q::value_index(c, 4 * q)) >> 2;
        f32x4 v = lds4[Q::swz(unit)];
        if (!valid) v = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
        xr[4 * q + 0] = v.x; xr[4 * q + 1] = v.y; xr[4 * q + 2] = v.z; xr[4 * q + 3] = v.w;
        sx[Q::sum_index(4 * q)] += (v.x + v.y) + (v.z + v.w);
      }
      const uint8_t* col = w + static_cast<size_t>(sbc) * Q::SB;
      for (u32 b = 0; b < batches; ++b) {
        const u32 rl = (b * groups + grp) * U;
        typename Q::Regs regs[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
          u32 row = row0 + rl + u;
          row = row < n_dim ? row : n_dim - 1;
          Q::load(regs[u], col + row * row_bytes, c);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const float p = wave_sum(Q::dot(regs[u], c, xr, sx));
          if (lane == 0) {
            const u32 idx = sw * rows_per_block + rl + u;
            part[idx] = (slab == sw) ? p : part[idx] + p;
          }
        }
      }
    }
  }
  __syncthreads();
  for (u32 t = tid; t < rows_per_block; t += blockDim.x) {
    const u32 row = row0 + t;
    if (row < n_dim) {
      float s = part[t];
      for (u32 i = 1; i < sw_count; ++i) s += part[i * rows_per_block + t];
      y[row] = s;
    }
  }
}

// ------------------------------------------------------------------------------------------
// Generic GEMV body: one wave per row, byte loads only.  Any pointer alignment, any K that is
// a multiple of 256, no LDS.  The slow path behind the fast kernels' alignment preconditions.
// ------------------------------------------------------------------------------------------
template <int FMT, int POLICY>
__device__ __forceinline__ void gemv_generic_body(float* __restrict__ y, const uint8_t* __restrict__ w,
                                                  const float* __restrict__ x, u32 k_dim, u32 n_dim,
                                                  u32 block_id, u32 num_blocks) {
  constexpr u32 SB = sb_bytes<FMT>::value;
  const u32 lane = threadIdx.x & 63u, wave = threadIdx.x >> 6, waves = blockDim.x >> 6;
  if (waves == 0) return;
  const u32 nsb = k_dim >> 8;
  for (u32 row = block_id * waves + wave; row < n_dim; row += num_blocks * waves) {
    const uint8_t* rp = w + static_cast<size_t>(row) * nsb * SB;
    float acc = 0.0f;
    for (u32 s = 0; s < nsb; ++s) {
      const uint8_t* bp = rp + static_cast<size_t>(s) * SB;
#pragma unroll
      for (u32 t = 0; t < 4; ++t) {
        const u32 i = lane + 64u * t;
        acc = fmaf(decode_value<FMT, POLICY>(bp, i), x[256u * s + i], acc);
      }
    }
    acc = wave_sum(acc);
    if (lane == 0) y[row] = acc;
  }
}

#define KQ_GEMV_KERNELS(fmtname, FMT)                                                                    \
  extern "C" __global__ void __launch_bounds__(512)                                                      \
      fmtname##_gemv_warp_reduce(float* y, const uint8_t* w, const float* x, u32 k_dim, u32 n_dim) {     \
    gemv_fast_body<FMT, 2>(y, w, x, k_dim, n_dim, blockIdx.x, gridDim.x);                                \
  }                                                                                                      \
  extern "C" __global__ void __launch_bounds__(256)                                                      \
      fmtname##_gemv_generic(float* y, const uint8_t* w, const float* x, u32 k_dim, u32 n_dim) {         \
    gemv_generic_body<FMT, POLICY_GEMV>(y, w, x, k_dim, n_dim, blockIdx.x, gridDim.x);                   \
  }

KQ_GEMV_KERNELS(q4k, FMT_Q4K)
KQ_GEMV_KERNELS(q5k, FMT_Q5K)
KQ_GEMV_KERNELS(q6k, FMT_Q6K)

// ------------------------------------------------------------------------------------------
// Batched GEMM  C[m x n] = A[m x k] . dequant(W[n x k])^T,  c[row*n + col] (quantize.rs:568-574).
// The contraction is the intended one (a dot product per (row, col)), with the GEMV-family
// decode, so m = 1 equals the GEMV.  VALU form: blockIdx.y walks the rows of A.
// ------------------------------------------------------------------------------------------
#define KQ_GEMM_KERNELS(fmtname, FMT)                                                                    \
  extern "C" __global__ void __launch_bounds__(512)                                                      \
      fmtname##_gemm_ggml(const float* a, const uint8_t* b_quant, float* c, u32 m, u32 n, u32 k) {       \
    for (u32 r = blockIdx.y; r < m; r += gridDim.y) {                                                    \
      gemv_fast_body<FMT, 2>(c + static_cast<size_t>(r) * n, b_quant, a + static_cast<size_t>(r) * k,    \
                             k, n, blockIdx.x, gridDim.x);                                               \
      __syncthreads();                                                                                   \
    }                                                                                                    \
  }                                                                                                      \
  extern "C" __global__ void __launch_bounds__(256)                                                      \
      fmtname##_gemm_generic(const float* a, const uint8_t* b_quant, float* c, u32 m, u32 n, u32 k) {    \
    for (u32 r = blockIdx.y; r < m; r += gridDim.y)                                                      \
      gemv_generic_body<FMT, POLICY_GEMV>(c + static_cast<size_t>(r) * n, b_quant,                       \
                                          a + static_cast<size_t>(r) * k, k, n, blockIdx.x, gridDim.x);  \
  }

KQ_GEMM_KERNELS(q4k, FMT_Q4K)
KQ_GEMM_KERNELS(q5k, FMT_Q5K)
KQ_GEMM_KERNELS(q6k, FMT_Q6K)

// ------------------------------------------------------------------------------------------
// Dequantise to f32 (test surface): out[sb*256 + i] = w_i.  The fast form shares load/unpack
// with the GEMV; the generic form takes the decode policy (0 = GEMV family, 1 = GEMM family as
// written in the reference) and any alignment.
// ------------------------------------------------------------------------------------------
template <int FMT>
__device__ __forceinline__ void dequant_fast_body(float* __restrict__ out, const uint8_t* __restrict__ w, uint64_t n_sb) {
  using Q = Quarter<FMT>;
  const uint64_t stride = static_cast<uint64_t>(gridDim.x) * blockDim.x;
  for (uint64_t gid = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x; gid < n_sb * 4; gid += stride) {
    const uint64_t sb = gid >> 2;
    const u32 c = static_cast<u32>(gid & 3u);
    typename Q::Regs r;
    Q::load(r, w + sb * Q::SB, c);
    float wv[64];
    Q::dequant(r, c, wv);
    float* o = out + sb * 256;
#pragma unroll
    for (int q = 0; q < 16; ++q) {
      f32x4 v = {wv[4 * q], wv[4 * q + 1], wv[4 * q + 2], wv[4 * q + 3]};
      *reinterpret_cast<f32x4*>(o + Q::value_index(c, 4 * q)) = v;
    }
  }
}

template <int FMT>
__device__ __forceinline__ void dequant_generic_body(float* __restrict__ out, const uint8_t* __restrict__ w,
                                                     uint64_t n_sb, int policy) {
  constexpr u32 SB = sb_bytes<FMT>::value;
  const uint64_t stride = static_cast<uint64_t>(gridDim.x) * blockDim.x;
  for (uint64_t gid = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x; gid < n_sb * 256; gid += stride) {
    const uint8_t* bp = w + (gid >> 8) * SB;
    const u32 i = static_cast<u32>(gid & 255u);
    out[gid] = policy == POLICY_GEMV ? decode_value<FMT, POLICY_GEMV>(bp, i) : decode_value<FMT, POLICY_GEMM_LEGACY>(bp, i);
  }
}

#define KQ_DEQUANT_KERNELS(fmtname, FMT)                                                                 \
  extern "C" __global__ void __launch_bounds__(256)                                                      \
      fmtname##_dequant_f32(float* out, const uint8_t* w, uint64_t n_sb) {                               \
    dequant_fast_body<FMT>(out, w, n_sb);                                                                \
  }                                                                                                      \
  extern "C" __global__ void __launch_bounds__(256)                                                      \
      fmtname##_dequant_f32_generic(float* out, const uint8_t* w, uint64_t n_sb, int policy) {           \
    dequant_generic_body<FMT>(out, w, n_sb, policy);                                                     \
  }

KQ_DEQUANT_KERNELS(q4k, FMT_Q4K)
KQ_DEQUANT_KERNELS(q5k, FMT_Q5K)
KQ_DEQUANT_KERNELS(q6k, FMT_Q6K)

// Plain copy, 16 bytes per lane: the yardstick the HBM counters are scaled by.
extern "C" __global__ void __launch_bounds__(256) kq_copy_u128(u32x4* dst, const u32x4* src, uint64_t n) {
  const uint64_t stride = static_cast<uint64_t>(gridDim.x) * blockDim.x;
  for (uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += stride) dst[i] = src[i];
}
