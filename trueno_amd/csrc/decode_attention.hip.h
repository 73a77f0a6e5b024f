// Single-query attention over a KV cache for autoregressive decoding (trueno-gpu/src/kernels/attention.rs:808-1095,
// IncrementalAttentionKernel, kernel name "incremental_attention"):
//   out[h][:] = sum_i softmax_i(scale * q[h] . k[kv(h)][i]) * v[kv(h)][i],  i < seq_len,  kv(h) = h * num_kv_heads / num_heads
//   q, out: [num_heads][head_dim];  k, v: [num_kv_heads][max_seq_len][head_dim];  f32.
// The reference walks the positions one by one in a single warp per head with an online softmax (Milakov &
// Gimelshein) and two elements per lane, which covers head_dim <= 64; this kernel computes the same function for
// head_dim up to 256.  Bound by HBM: K and V are read once, 8 * num_kv_heads * seq_len * head_dim bytes.
//
// A position's row of K (and of V) is read by head_dim/4 lanes with one 128-bit load each, so a wave takes
// 64 / (head_dim/4) positions at a time; each such lane group keeps its own running (max, sum, output) over the
// positions it sees.  The positions of a head are cut in chunks over the grid and a chunk over the 4 waves of a
// workgroup; groups, waves and chunks are merged with the usual rescaling, the chunks through memory by the
// workgroup that arrives last at the head's counter (in chunk order: the same bits on every run).  Exponentials
// are 2^x on scores pre-multiplied by log2(e), as in the reference (ex2.approx there, v_exp_f32 here).
#pragma once
#include "kquant_common.hip.h"

namespace decode_attention {

constexpr u32 kWaves = 4;
constexpr float kLog2e = 1.4426950408889634f;

struct State {          // running softmax over some positions, in the 2^x domain
  float m, s;
  f32x4 o;
};

__device__ __forceinline__ void merge(State& a, float m, float s, const f32x4& o) {
  // one of the two factors is always 1: a single exponential, of (smaller maximum - larger maximum)
  const bool keep = a.m >= m;
  const float nm = keep ? a.m : m, other = keep ? m : a.m;
  const float e = other == nm ? 1.0f : __builtin_amdgcn_exp2f(other - nm);  // -inf - -inf never reaches exp2
  const float ca = keep ? 1.0f : e, cb = keep ? e : 1.0f;
  a.s = a.s * ca + s * cb;
  a.o.x = a.o.x * ca + o.x * cb; a.o.y = a.o.y * ca + o.y * cb;
  a.o.z = a.o.z * ca + o.z * cb; a.o.w = a.o.w * ca + o.w * cb;
  a.m = nm;
}

// Sum of v over each group of 2^lpp_log2 neighbouring lanes, in every lane of the group, without going through LDS
// (five dependent ds_bpermute per position cost more than the position's memory traffic): DPP within a row of 16
// lanes, row sums through SGPRs beyond that.
__device__ __forceinline__ float group_sum(float v, u32 lpp_log2, u32 lane) {
  if (lpp_log2 >= 1u) v += dpp_f32<0xB1>(v);    // quad_perm [1,0,3,2]
  if (lpp_log2 >= 2u) v += dpp_f32<0x4E>(v);    // quad_perm [2,3,0,1]
  if (lpp_log2 >= 3u) v += dpp_f32<0x141>(v);   // row_half_mirror
  if (lpp_log2 >= 4u) v += dpp_f32<0x140>(v);   // row_mirror: every lane of a row of 16 holds the row's sum
  if (lpp_log2 >= 5u) {
    const float r0 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0));
    const float r1 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 16));
    const float r2 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32));
    const float r3 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 48));
    const float lo = r0 + r1, hi = r2 + r3;
    v = lpp_log2 >= 6u ? lo + hi : (lane < 32u ? lo : hi);
  }
  return v;
}

// lanes per position LPP = 2^lpp_log2 >= head_dim / 4
__device__ __forceinline__ void body(const float* __restrict__ q, const float* __restrict__ k, const float* __restrict__ v,
                                     float* __restrict__ out, u32 seq_len, u32 head_dim, u32 num_heads, u32 num_kv_heads,
                                     u32 max_seq_len, float scale, u32 lpp_log2, u32 chunk, u32 chunks,
                                     float* __restrict__ partial, u32* __restrict__ counters) {
  __shared__ float s_m[kWaves][64], s_s[kWaves][64];
  __shared__ f32x4 s_o[kWaves][64];
  __shared__ u32 s_old;
  const u32 lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
  const u32 head = blockIdx.x / chunks, ci = blockIdx.x - head * chunks;
  const u32 kv_head = static_cast<u32>((static_cast<uint64_t>(head) * num_kv_heads) / num_heads);
  const u32 lpp = 1u << lpp_log2, ppw = 64u >> lpp_log2;           // lanes per position, positions per wave and step
  const u32 sub = lane & (lpp - 1u), grp = lane >> lpp_log2;
  const bool live = 4u * sub < head_dim;                             // head_dim % 4 == 0
  const size_t kv_base = static_cast<size_t>(kv_head) * max_seq_len * head_dim;
  const f32x4 zero4 = {0.0f, 0.0f, 0.0f, 0.0f};
  // the chunks' states cross workgroups (and XCDs): 16-byte buffer accesses at agent scope (sc1)
  const __amdgpu_buffer_rsrc_t part_rsrc =
      __builtin_amdgcn_make_buffer_rsrc(partial, 0, static_cast<int>(min(static_cast<size_t>(0x7FFFFFFF), static_cast<size_t>(num_heads) * chunks * lpp * 32u)), 0x00020000);
  const f32x4 qv = live ? reinterpret_cast<const f32x4*>(q + static_cast<size_t>(head) * head_dim)[sub] : zero4;
  const float sl = scale * kLog2e;
  const u32 p0 = ci * chunk, p1 = min(seq_len, p0 + chunk);
  State st = {-INFINITY, 0.0f, zero4};
  constexpr u32 kAhead = 4;                     // positions per lane group whose rows are in flight together
  const u32 stride = kWaves * ppw;
  for (u32 p = p0 + wave * ppw + grp; p < p1; p += kAhead * stride) {
    f32x4 kk[kAhead], vv[kAhead];
#pragma unroll
    for (u32 a = 0; a < kAhead; ++a) {
      const u32 pa = min(p + a * stride, p1 - 1u);          // clamped: read, then ignored
      const size_t row = kv_base + static_cast<size_t>(pa) * head_dim;
      // (the cache is read once per call, a row in whole lines: the non-temporal hint is worth 3-11 % here)
      kk[a] = live ? __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(k + row) + sub) : zero4;
      vv[a] = live ? __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(v + row) + sub) : zero4;
    }
#pragma unroll
    for (u32 a = 0; a < kAhead; ++a) {
      float d = fmaf(qv.w, kk[a].w, fmaf(qv.z, kk[a].z, fmaf(qv.y, kk[a].y, qv.x * kk[a].x)));
      d = group_sum(d, lpp_log2, lane);
      if (p + a * stride < p1) merge(st, d * sl, 1.0f, vv[a]);
    }
  }
  // the lane groups of a wave, then the waves of the workgroup: lane `sub` of group 0 ends up with the chunk's state
  for (u32 off = lpp; off < 64u; off <<= 1) {
    const float m = __shfl_xor(st.m, off, 64), s = __shfl_xor(st.s, off, 64);
    f32x4 o;
    o.x = __shfl_xor(st.o.x, off, 64); o.y = __shfl_xor(st.o.y, off, 64);
    o.z = __shfl_xor(st.o.z, off, 64); o.w = __shfl_xor(st.o.w, off, 64);
    merge(st, m, s, o);
  }
  s_m[wave][lane] = st.m; s_s[wave][lane] = st.s; s_o[wave][lane] = st.o;
  __syncthreads();
  if (wave != 0u || lane >= lpp) {
    if (chunks == 1u) return;
  } else {
    for (u32 w = 1; w < kWaves; ++w) merge(st, s_m[w][lane], s_s[w][lane], s_o[w][lane]);
    float* dst = out + static_cast<size_t>(head) * head_dim + 4u * sub;
    if (chunks == 1u) {
      if (live) {
        const float inv = 1.0f / st.s;
        *reinterpret_cast<f32x4*>(dst) = f32x4{st.o.x * inv, st.o.y * inv, st.o.z * inv, st.o.w * inv};
      }
      return;
    }
    // [head][chunk][lpp lanes][m, s, -, -, o.xyzw] through to memory: two 16-byte stores at agent scope
    const u32 slot = static_cast<u32>(((static_cast<size_t>(head) * chunks + ci) * lpp + sub) * 32u);
    __builtin_amdgcn_raw_buffer_store_b128(u32x4{__float_as_uint(st.m), __float_as_uint(st.s), 0u, 0u}, part_rsrc, static_cast<int>(slot), 0, 16);
    __builtin_amdgcn_raw_buffer_store_b128(u32x4{__float_as_uint(st.o.x), __float_as_uint(st.o.y), __float_as_uint(st.o.z), __float_as_uint(st.o.w)},
                                           part_rsrc, static_cast<int>(slot + 16u), 0, 16);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if (lane == 0u) {
      const u32 old = __hip_atomic_fetch_add(counters + head, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (old == chunks - 1u) __hip_atomic_store(counters + head, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      s_old = old;
    }
  }
  __syncthreads();
  if (wave != 0u || lane >= lpp || s_old != chunks - 1u) return;
  State tot = {-INFINITY, 0.0f, zero4};
  constexpr u32 kRound = 16;                       // chunks whose states are in flight together; merged in chunk order
  for (u32 c0 = 0; c0 < chunks; c0 += kRound) {
    u32x4 ms[kRound], ov[kRound];
#pragma unroll
    for (u32 cc = 0; cc < kRound; ++cc) {
      const u32 c = min(c0 + cc, chunks - 1u);
      const u32 slot = static_cast<u32>(((static_cast<size_t>(head) * chunks + c) * lpp + sub) * 32u);
      ms[cc] = __builtin_amdgcn_raw_buffer_load_b128(part_rsrc, static_cast<int>(slot), 0, 16);
      ov[cc] = __builtin_amdgcn_raw_buffer_load_b128(part_rsrc, static_cast<int>(slot + 16u), 0, 16);
    }
#pragma unroll
    for (u32 cc = 0; cc < kRound; ++cc)
      if (c0 + cc < chunks)
        merge(tot, __uint_as_float(ms[cc].x), __uint_as_float(ms[cc].y),
              f32x4{__uint_as_float(ov[cc].x), __uint_as_float(ov[cc].y), __uint_as_float(ov[cc].z), __uint_as_float(ov[cc].w)});
  }
  if (live) {
    const float inv = 1.0f / tot.s;
    *reinterpret_cast<f32x4*>(out + static_cast<size_t>(head) * head_dim + 4u * sub) =
        f32x4{tot.o.x * inv, tot.o.y * inv, tot.o.z * inv, tot.o.w * inv};
  }
}

}  // namespace decode_attention
