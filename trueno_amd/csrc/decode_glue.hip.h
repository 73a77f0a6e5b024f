// The element-wise steps between the GEMVs of a decoder layer (trueno-gpu/src/kernels/elementwise.rs and
// layernorm.rs): residual add, RMSNorm, residual add + RMSNorm, SwiGLU.  f32 in, f32 out, a few KB each: they
// are bound by launch and memory latency, not by bandwidth.
//
// Arithmetic follows the reference's instruction sequences (every mul/add/div its own IEEE rounding, the sum of
// squares by fma); only the summation order of the sum of squares (256 threads here, 32 there) and the two
// approximate instructions differ in the last bits: the reference uses PTX ex2.approx / rsqrt.approx (documented
// to 2^-22 relative), here v_exp_f32 / v_rsq_f32 (1 ulp).
#pragma once
#include "kquant_common.hip.h"

namespace glue {

// output[i] = input1[i] + input2[i]   (elementwise.rs:33-101; output may alias an input)
__device__ __forceinline__ void residual_add_body(const float* in1, const float* in2, float* out, u32 n) {
  for (u32 i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x) out[i] = __fadd_rn(in1[i], in2[i]);
}

// output[i] = (gate[i] * sigmoid(gate[i])) * up[i],  sigmoid(g) = 1 / (1 + 2^(-g * 1.442695f))   (elementwise.rs:521-592)
__device__ __forceinline__ void fused_swiglu_body(const float* gate, const float* up, float* out, u32 n) {
  for (u32 i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x) {
    const float g = gate[i];
    const float scaled = __fmul_rn(__fsub_rn(0.0f, g), 1.442695f);
    const float denom = __fadd_rn(1.0f, __builtin_amdgcn_exp2f(scaled));
    const float sigmoid = __fdiv_rn(1.0f, denom);
    out[i] = __fmul_rn(__fmul_rn(g, sigmoid), up[i]);
  }
}

// Sum over the workgroup (up to 16 waves): the waves' sums are added in wave order.
__device__ __forceinline__ float block_sum(float v, float* s_part) {
  v = wave_sum(v);
  const u32 wave = threadIdx.x >> 6, waves = (blockDim.x + 63u) >> 6;
  if ((threadIdx.x & 63u) == 0u) s_part[wave] = v;
  __syncthreads();
  float total = s_part[0];
  for (u32 w = 1; w < waves; ++w) total += s_part[w];
  __syncthreads();
  return total;
}

// One row: output[i] = (x[i] * rsqrt(mean(x^2) + eps)) * gamma[i] with x = input, or x = residual + input
// (layernorm.rs:388-516, elementwise.rs:109-248).  One workgroup; output may alias input (residual).  With a
// residual the sums x are parked in `output` between the two passes, as the reference does; a thread only ever
// re-reads what it wrote itself.
template <bool RESIDUAL>
__device__ __forceinline__ void rmsnorm_body(const float* residual, const float* in, float* out, const float* gamma,
                                             u32 hidden, float eps) {
  __shared__ float s_part[16];
  float sq = 0.0f;
  for (u32 i = threadIdx.x; i < hidden; i += blockDim.x) {
    float x = in[i];
    if constexpr (RESIDUAL) {
      x = __fadd_rn(residual[i], x);
      out[i] = x;
    }
    sq = fmaf(x, x, sq);
  }
  const float total = block_sum(sq, s_part);
  const float mean_sq = __fdiv_rn(total, static_cast<float>(hidden));
  const float rms_inv = __builtin_amdgcn_rsqf(__fadd_rn(mean_sq, eps));
  for (u32 i = threadIdx.x; i < hidden; i += blockDim.x) {
    const float x = RESIDUAL ? out[i] : in[i];
    out[i] = __fmul_rn(__fmul_rn(x, rms_inv), gamma[i]);
  }
}

}  // namespace glue
