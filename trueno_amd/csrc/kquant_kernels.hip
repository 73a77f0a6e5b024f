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
#ifndef KQ_U
#define KQ_U 2      // rows a wave of the fast GEMV engine has in flight (the host's kGemvRowsPerBatch)
#endif
#include "kquant_chain.hip.h"
#include "kquant_gemm_f16.hip.h"
#include "kquant_few_i8.hip.h"
#include "decode_glue.hip.h"
#include "gemv_f32.hip.h"
#include "decode_attention.hip.h"

// The fast GEMV engine is chain_step() of kquant_chain.hip.h: one workgroup owns a run of rows; the
// activation vector is staged once into LDS (swizzled), each wave keeps its 64-activations-per-lane
// slice in registers and streams rows (U rows of 128-bit loads in flight per wave), unpacks in
// registers, forms the factorised dot product and reduces across the wave with DPP.  K is cut in
// slabs of 16 super-blocks (one wave-width); with S slabs, min(S, waves) waves share a row and
// their partial sums meet in LDS.
//   dynamic LDS = K*4 (activations) + Sw*R*4 (partial sums) + 64 bytes

// ------------------------------------------------------------------------------------------
// Generic GEMV body: one wave per row, byte loads only.  Any pointer alignment, any K that is
// a multiple of 256, no LDS.  The slow path behind the fast kernels' alignment preconditions.
// ------------------------------------------------------------------------------------------
template <int FMT, int POLICY>
__device__ __forceinline__ void gemv_generic_body(float* __restrict__ y, const uint8_t* __restrict__ w,
                                                  const float* __restrict__ x, u32 k_dim, u32 n_dim,
                                                  u32 block_id, u32 num_blocks, u32 flags) {
  constexpr u32 SB = sb_bytes<FMT>::value;
  const u32 lane = threadIdx.x & 63u, wave = threadIdx.x >> 6, waves = blockDim.x >> 6;
  if (waves == 0) return;
  const u32 nsb = k_dim >> 8;
  float scale = 1.0f;
  if (flags & CHAIN_NORM_INPUT) {
    float total = 0.0f;   // the fixed order of kquant_chain.hip.h: groups of 64 units, butterfly within, in order across
    for (u32 g = 0; g < nsb; ++g) {
      const f32x4 v = {x[256u * g + 4u * lane], x[256u * g + 4u * lane + 1u], x[256u * g + 4u * lane + 2u], x[256u * g + 4u * lane + 3u]};
      const float sg = wave_sum(unit_sumsq(v));
      total = g == 0u ? sg : total + sg;
    }
    scale = 1.0f / sqrtf(total / static_cast<float>(k_dim) + kChainNormEps);
  }
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
    if (lane == 0) y[row] = acc * scale;
  }
}

#define KQ_GEMV_KERNELS(fmtname, FMT)                                                                    \
  extern "C" __global__ void __launch_bounds__(768)                                                      \
      fmtname##_gemv_warp_reduce(float* y, const uint8_t* w, const float* x, u32 k_dim, u32 n_dim) {     \
    extern __shared__ f32x4 lds4[];                                                                      \
    __shared__ u32 s_flag;                                                                               \
    const ChainEntry e = {FMT, k_dim, n_dim, 0u, w, x, y};                                               \
    chain_step<FMT, KQ_U>(e, nullptr, 0u, nullptr, lds4, &s_flag, blockIdx.x, gridDim.x, blockDim.x);                                          \
  }                                                                                                      \
  extern "C" __global__ void __launch_bounds__(768)                                                      \
      fmtname##_gemv_flags(float* y, const uint8_t* w, const float* x, u32 k_dim, u32 n_dim, u32 flags) {\
    extern __shared__ f32x4 lds4[];                                                                      \
    __shared__ u32 s_flag;                                                                               \
    const ChainEntry e = {FMT, k_dim, n_dim, flags, w, x, y};                                            \
    chain_step<FMT, KQ_U>(e, nullptr, 0u, nullptr, lds4, &s_flag, blockIdx.x, gridDim.x, blockDim.x);                                          \
  }                                                                                                      \
  extern "C" __global__ void __launch_bounds__(256)                                                      \
      fmtname##_gemv_generic(float* y, const uint8_t* w, const float* x, u32 k_dim, u32 n_dim, u32 flags) { \
    gemv_generic_body<FMT, POLICY_GEMV>(y, w, x, k_dim, n_dim, blockIdx.x, gridDim.x, flags);            \
  }

KQ_GEMV_KERNELS(q4k, FMT_Q4K)
KQ_GEMV_KERNELS(q5k, FMT_Q5K)
KQ_GEMV_KERNELS(q6k, FMT_Q6K)

// Up to sixteen GEMVs that do not depend on one another (the q, k, v projections of a decoder layer; gate and
// up; entries of neighbouring layers where a list allows it) in one launch: consecutive runs of workgroups belong to
// consecutive entries.  Each entry is computed exactly as its own launch would compute it.
// A workgroup can ask for its first rows only once it knows its matrix, and kernel arguments come from memory: finding
// the entry through a table in the argument and then reading the entry would be two memory round trips in a row.  The
// table therefore travels as eight leading scalar arguments, which the build asks the hardware to place in scalar
// registers when a wave starts (kernel-argument preload); the entry is then one indexed read, whose `hot` part is all
// that the first loads need.
struct GemvGroupHot {
  const uint8_t* w;
  const float* x;
  u32 k, n, fmt, flags;
  u32 first_block, num_blocks;      // the entry's run of workgroups
};
struct GemvGroupCold {
  float* y;
  const float* gamma;
  const float* x2;
  const float* residual;
  float eps;
  u32 pad;
};
constexpr u32 kGroupEntries = 16;
struct GemvGroup {
  GemvGroupHot hot[kGroupEntries];
  GemvGroupCold cold[kGroupEntries];
};
// firsts: first[j], j = 1 .. 16, is the first workgroup of entry j (entries that do not exist, and first[16], repeat the
// grid size), two to an argument: first[2a + 1] in the low half of argument a, first[2a + 2] in the high half (a grid has
// fewer than 65536 workgroups).  The entry of a workgroup is the last one that starts at or before it: four compares.
extern "C" __global__ void __launch_bounds__(768)
kq_gemv_group(u32 firsts0, u32 firsts1, u32 firsts2, u32 firsts3, u32 firsts4, u32 firsts5, u32 firsts6, u32 firsts7, const GemvGroup g) {
  extern __shared__ f32x4 lds4[];
  __shared__ u32 s_flag;
  const u32 b = blockIdx.x;
  u32 i = b >= (firsts3 >> 16) ? 8u : 0u;                                               // first[8]
  i += b >= ((i ? firsts5 : firsts1) >> 16) ? 4u : 0u;                                  // first[12], first[4]
  const u32 p2 = (i & 8u) ? ((i & 4u) ? firsts6 : firsts4) : ((i & 4u) ? firsts2 : firsts0);      // first[i + 2]
  i += b >= (p2 >> 16) ? 2u : 0u;
  // first[i + 1]: the low half of argument i / 2, picked bit by bit (selects, no branches)
  const u32 q0 = (i & 8u) ? firsts4 : firsts0, q1 = (i & 8u) ? firsts5 : firsts1, q2 = (i & 8u) ? firsts6 : firsts2,
            q3 = (i & 8u) ? firsts7 : firsts3;
  const u32 r0 = (i & 4u) ? q2 : q0, r1 = (i & 4u) ? q3 : q1;
  const u32 p1 = (i & 2u) ? r1 : r0;
  i += b >= (p1 & 0xFFFFu) ? 1u : 0u;
  GemvGroupHot h = g.hot[i];
  const GemvGroupCold c = g.cold[i];
  // the block size is an implicit kernel argument, a load like the entry's: all of them in flight together, one wait
  u32 block_threads = blockDim.x;
  asm volatile("" : "+s"(block_threads), "+s"(h.k), "+s"(h.flags));
  const ChainEntry e = {h.fmt, h.k, h.n, h.flags, h.w, h.x, c.y, c.gamma, c.x2, c.residual, c.eps, 0u};
  const u32 block_id = b - h.first_block, num_blocks = h.num_blocks;
  if (e.fmt == FMT_Q4K) chain_step<FMT_Q4K, KQ_U>(e, nullptr, 0u, nullptr, lds4, &s_flag, block_id, num_blocks, block_threads);
  else if (e.fmt == FMT_Q5K) chain_step<FMT_Q5K, KQ_U>(e, nullptr, 0u, nullptr, lds4, &s_flag, block_id, num_blocks, block_threads);
  else if (e.fmt == FMT_Q6K) chain_step<FMT_Q6K, KQ_U>(e, nullptr, 0u, nullptr, lds4, &s_flag, block_id, num_blocks, block_threads);
}

// Any number of GEMVs that do not depend on one another in one launch of one workgroup per place on the chip: the
// launcher cuts the entries' rows into items (entry, first row, rows) of equal cost per workgroup, in list order, so a
// workgroup takes the end of one entry and the beginning of the next - or a slice of a large one - and all of them end
// together; with many entries to a launch the fixed time of a launch (its first bytes arrive slowly, its last
// workgroups run alone) is paid once for gigabytes.  Tables in device memory: wgs[2 b] = first item of workgroup b,
// wgs[2 b + 1] = its number of items.  An item is computed exactly as a workgroup of a launch of its own would.
struct GemvItem { u32 entry, row0, rows, pad; };
// items i .. of this workgroup for as long as they are of format FMT (one loop per format: with the three engines side
// by side in one loop body the register allocator needs half again as many registers)
template <int FMT>
__device__ __forceinline__ u32 many_run(u32 i, u32 count, const GemvItem* __restrict__ items, const GemvGroupHot* __restrict__ hot,
                                        const GemvGroupCold* __restrict__ cold, f32x4* lds4, u32* s_flag, u32 block_threads) {
  for (; i < count; ++i) {
    const GemvItem it = items[i];
    const GemvGroupHot h = hot[it.entry];
    if (h.fmt != static_cast<u32>(FMT)) break;
    const GemvGroupCold c = cold[it.entry];
    const ChainEntry e = {h.fmt, h.k, h.n, h.flags, h.w, h.x, c.y, c.gamma, c.x2, c.residual, c.eps, 0u};
    chain_step_rows<FMT, KQ_U>(e, nullptr, 0u, nullptr, lds4, s_flag, it.row0, it.rows, block_threads);
    __syncthreads();      // the next item's vector goes where this one's partial sums are still being read
  }
  return i;
}
extern "C" __global__ void __launch_bounds__(768)
kq_gemv_many(const u32* __restrict__ wgs, const GemvItem* __restrict__ items, const GemvGroupHot* __restrict__ hot,
             const GemvGroupCold* __restrict__ cold) {
  extern __shared__ f32x4 lds4[];
  __shared__ u32 s_flag;
  const u32 count = wgs[2u * blockIdx.x + 1u];
  items += wgs[2u * blockIdx.x];
  const u32 block_threads = blockDim.x;
  u32 i = 0;
  while (i < count) {
    const u32 fmt = hot[items[i].entry].fmt;
    if (fmt == FMT_Q4K) i = many_run<FMT_Q4K>(i, count, items, hot, cold, lds4, &s_flag, block_threads);
    else if (fmt == FMT_Q5K) i = many_run<FMT_Q5K>(i, count, items, hot, cold, lds4, &s_flag, block_threads);
    else if (fmt == FMT_Q6K) i = many_run<FMT_Q6K>(i, count, items, hot, cold, lds4, &s_flag, block_threads);
    else ++i;
  }
}

// The list as phases of independent entries in one resident launch, one workgroup of 12 waves per CU.
extern "C" __global__ void __launch_bounds__(768)
kq_gemv_phases(const ChainEntry* entries, const PhaseAssign* assign, u32 phases, u32* counters, u32* status, u32 spin_limit) {
  phases_body<KQ_U>(entries, assign, phases, counters, status, spin_limit);
}

// ------------------------------------------------------------------------------------------
// Element-wise steps of a decoder layer under the reference's kernel names (decode_glue.hip.h).  residual_add and
// fused_swiglu keep the reference's parameter lists (elementwise.rs:56-59, 541-544).  The reference compiles the
// row length and epsilon of rmsnorm / fused_residual_rmsnorm into the PTX (layernorm.rs:424-431,
// elementwise.rs:145-149); with one pre-built code object they are two more parameters after the pointers.
// ------------------------------------------------------------------------------------------
extern "C" __global__ void __launch_bounds__(256) residual_add(const float* input1, const float* input2, float* output, u32 n) {
  glue::residual_add_body(input1, input2, output, n);
}
extern "C" __global__ void __launch_bounds__(256) fused_swiglu(const float* gate, const float* up, float* output, u32 n) {
  glue::fused_swiglu_body(gate, up, output, n);
}
extern "C" __global__ void __launch_bounds__(1024)
rmsnorm(const float* input, float* output, const float* gamma, u32 hidden_size, float epsilon) {
  glue::rmsnorm_body<false>(nullptr, input, output, gamma, hidden_size, epsilon);
}
extern "C" __global__ void __launch_bounds__(1024)
fused_residual_rmsnorm(const float* residual, const float* input, float* output, const float* gamma, u32 hidden_size, float epsilon) {
  glue::rmsnorm_body<true>(residual, input, output, gamma, hidden_size, epsilon);
}

// f32 GEMV under the reference's two kernel names and parameter list (gemv.rs:53-57, 222-226): one engine
// (gemv_f32.hip.h), the two names differ only in the reference's summation order.  gemv_f32_fast takes the
// launcher's extra arguments; the named kernels are the any-shape form.
extern "C" __global__ void __launch_bounds__(512)
gemv_f32_fast(float* y, const float* a, const float* x, float* partial, u32* counters, u32 k_dim, u32 n_dim, u32 rows_per_part,
              u32 parts) {
  gemv_f32::fast_body(y, a, x, partial, counters, k_dim, n_dim, rows_per_part, parts);
}
extern "C" __global__ void __launch_bounds__(256) gemv_warp_reduce(float* y, const float* a, const float* x, u32 k_dim, u32 n_dim) {
  gemv_f32::generic_body(y, a, x, k_dim, n_dim);
}
extern "C" __global__ void __launch_bounds__(256) gemv_coalesced(float* y, const float* a, const float* x, u32 k_dim, u32 n_dim) {
  gemv_f32::generic_body(y, a, x, k_dim, n_dim);
}

// GGML's Q5_K block (d, dmin, scales[12] packed as in Q4_K, qh[32], qs[128]; fifth bit of value 32 j + l in bit j of
// qh[l]) re-packed into the layout the reference's Q5_K kernels read (trueno-gpu/src/kernels/quantize.rs:1589-1693:
// d, dmin, eight contiguous 12-bit (scale, min) fields, qs[128] at 16, fifth bit of value i in bit i%8 of qh[i/8]
// at 144).  The dequantised values are the same, bit for bit.  One wave per block; dst may be src (a wave reads
// its whole block before it writes).
extern "C" __global__ void __launch_bounds__(256) q5k_from_ggml(uint8_t* dst, const uint8_t* src, uint64_t n_sb) {
  const u32 lane = threadIdx.x & 63u;
  const uint64_t wave = (static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x) >> 6;
  const uint64_t nwaves = (static_cast<uint64_t>(gridDim.x) * blockDim.x) >> 6;
  for (uint64_t sb = wave; sb < n_sb; sb += nwaves) {
    const uint8_t* in = src + sb * 176u;
    uint8_t* out = dst + sb * 176u;
    // everything this lane needs, before anything is written
    const u32 hdr = lane < 4u ? in[lane] : 0u;
    u32 sc[12];
#pragma unroll
    for (int i = 0; i < 12; ++i) sc[i] = in[4 + i];
    const u32 q0 = in[48u + 2u * lane], q1 = in[49u + 2u * lane];
    u32 hb = 0u;                       // lanes 0..31: byte `lane` of the new qh = values 8 lane .. 8 lane + 7
    if (lane < 32u) {
      const u32 j = lane >> 2, l0 = 8u * (lane & 3u);
#pragma unroll
      for (u32 b = 0; b < 8; ++b) hb |= ((static_cast<u32>(in[16u + l0 + b]) >> j) & 1u) << b;
    }
    u32 fb = 0u;                       // lanes 0..11: byte `lane` of the 96-bit string of 12-bit fields
    if (lane < 12u) {
#pragma unroll
      for (u32 b = 0; b < 8; ++b) {
        const u32 p = 8u * lane + b, j = p / 12u, r = p % 12u;
        u32 s6, m6;                    // get_scale_min_k4
        if (j < 4u) { s6 = sc[j] & 63u; m6 = sc[j + 4] & 63u; }
        else { s6 = (sc[j + 4] & 15u) | ((sc[j - 4] >> 6) << 4); m6 = (sc[j + 4] >> 4) | ((sc[j] >> 6) << 4); }
        fb |= (((r < 6u ? s6 >> r : m6 >> (r - 6u))) & 1u) << b;
      }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if (lane < 4u) out[lane] = static_cast<uint8_t>(hdr);
    if (lane < 12u) out[4u + lane] = static_cast<uint8_t>(fb);
    out[16u + 2u * lane] = static_cast<uint8_t>(q0);
    out[17u + 2u * lane] = static_cast<uint8_t>(q1);
    if (lane < 32u) out[144u + lane] = static_cast<uint8_t>(hb);
  }
}

// Single-query attention over the KV cache (decode_attention.hip.h) under the reference's kernel name.  The reference's
// parameter list is (q_ptr, k_ptr, v_ptr, out_ptr, seq_len) with head_dim, the head counts, max_seq_len and the scale
// compiled into the PTX (attention.rs:865-901); here they follow as parameters, then the launcher's own.
extern "C" __global__ void __launch_bounds__(256)
incremental_attention(const float* q, const float* k, const float* v, float* out, u32 seq_len, u32 head_dim, u32 num_heads,
                      u32 num_kv_heads, u32 max_seq_len, float scale, u32 lpp_log2, u32 chunk, u32 chunks, float* partial,
                      u32* counters) {
  decode_attention::body(q, k, v, out, seq_len, head_dim, num_heads, num_kv_heads, max_seq_len, scale, lpp_log2, chunk, chunks,
                         partial, counters);
}

extern "C" __global__ void __launch_bounds__(256) kq_fill_u32(u32* p, u32 n, u32 v) {
  for (u32 i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x) p[i] = v;
}

// ------------------------------------------------------------------------------------------
// Batched GEMM  C[m x n] = A[m x k] . dequant(W[n x k])^T,  c[row*n + col] (quantize.rs:568-574).
// The contraction is the intended one (a dot product per (row, col)), with the GEMV-family
// decode, so m = 1 equals the GEMV.  VALU form: blockIdx.y walks the rows of A.  *_gemm_as_written is the same
// product with the GEMM family's own decode as the reference writes it (quantize.rs:445-514, :727-807, :1009-1064:
// contiguous 12-bit scale fields normalised by 1/63, sequential nibbles, Q6_K's unsigned scales and ql + 4*q2),
// value by value, one wave per row of W.
// ------------------------------------------------------------------------------------------
#define KQ_GEMM_KERNELS(fmtname, FMT)                                                                    \
  extern "C" __global__ void __launch_bounds__(512)                                                      \
      fmtname##_gemm_ggml(const float* a, const uint8_t* b_quant, float* c, u32 m, u32 n, u32 k) {       \
    extern __shared__ f32x4 lds4[];                                                                      \
    __shared__ u32 s_flag;                                                                               \
    for (u32 r = blockIdx.y; r < m; r += gridDim.y) {                                                    \
      const ChainEntry e = {FMT, k, n, 0u, b_quant, a + static_cast<size_t>(r) * k,                      \
                            c + static_cast<size_t>(r) * n};                                             \
      chain_step<FMT, KQ_U>(e, nullptr, 0u, nullptr, lds4, &s_flag, blockIdx.x, gridDim.x, blockDim.x);                                        \
      __syncthreads();                                                                                   \
    }                                                                                                    \
  }                                                                                                      \
  extern "C" __global__ void __launch_bounds__(256)                                                      \
      fmtname##_gemm_generic(const float* a, const uint8_t* b_quant, float* c, u32 m, u32 n, u32 k) {    \
    for (u32 r = blockIdx.y; r < m; r += gridDim.y)                                                      \
      gemv_generic_body<FMT, POLICY_GEMV>(c + static_cast<size_t>(r) * n, b_quant,                       \
                                          a + static_cast<size_t>(r) * k, k, n, blockIdx.x, gridDim.x, 0u); \
  }                                                                                                      \
  extern "C" __global__ void __launch_bounds__(256)                                                      \
      fmtname##_gemm_as_written(const float* a, const uint8_t* b_quant, float* c, u32 m, u32 n, u32 k) { \
    for (u32 r = blockIdx.y; r < m; r += gridDim.y)                                                      \
      gemv_generic_body<FMT, POLICY_GEMM_LEGACY>(c + static_cast<size_t>(r) * n, b_quant,                \
                                                 a + static_cast<size_t>(r) * k, k, n, blockIdx.x, gridDim.x, 0u); \
  }

KQ_GEMM_KERNELS(q4k, FMT_Q4K)
KQ_GEMM_KERNELS(q5k, FMT_Q5K)
KQ_GEMM_KERNELS(q6k, FMT_Q6K)

// Matrix-core form of the k-quant GEMM for m >= 2 (kquant_gemm_f16.hip.h; the arguments: Geometry there).
#define KQ_GEMM_F16(name, threads, BODY)                                                                                \
  extern "C" __global__ void __launch_bounds__(threads)                                                                  \
  name(const float* a, const uint8_t* w, float* c, uint8_t* ws, u32 m, u32 n, u32 nsb, uint64_t geom) {                  \
    extern __shared__ uint8_t gemm_lds[];                                                                                \
    const u32 lds_base =                                                                                                 \
        static_cast<u32>(reinterpret_cast<size_t>((const __attribute__((address_space(3))) uint8_t*)gemm_lds));         \
    gemm_f16::BODY(a, w, c, ws, m, n, nsb, geom, lds_base);                                                              \
  }
#define KQ_COMMA ,
KQ_GEMM_F16(q4k_gemm_f16_w8, 512, kq_body<FMT_Q4K KQ_COMMA 8 KQ_COMMA 1>)
KQ_GEMM_F16(q4k_gemm_f16_w4, 256, kq_body<FMT_Q4K KQ_COMMA 4 KQ_COMMA 1>)
KQ_GEMM_F16(q4k_gemm_f16_w12, 768, kq_body<FMT_Q4K KQ_COMMA 12 KQ_COMMA 1>)
KQ_GEMM_F16(q5k_gemm_f16_w8, 512, kq_body<FMT_Q5K KQ_COMMA 8 KQ_COMMA 1>)
KQ_GEMM_F16(q5k_gemm_f16_w4, 256, kq_body<FMT_Q5K KQ_COMMA 4 KQ_COMMA 1>)
// two token tiles per workgroup (more than 16 tokens)
KQ_GEMM_F16(q4k_gemm_f16_w8t2, 512, kq_body<FMT_Q4K KQ_COMMA 8 KQ_COMMA 2>)
KQ_GEMM_F16(q5k_gemm_f16_w8t2, 512, kq_body<FMT_Q5K KQ_COMMA 8 KQ_COMMA 2>)
KQ_GEMM_F16(q6k_gemm_f16_w8, 512, q6k_body<1>)
KQ_GEMM_F16(q6k_gemm_f16_w4, 256, q6k_body<2>)

// Q4_K product for two to four tokens on the integer matrix cores (kquant_few_i8.hip.h): workgroup b takes the rows
// b * rows_per_wg .. of W, k <= 4096.
#define KQ_GEMM_FEW(name, NTOK)                                                                                          \
  extern "C" __global__ void __launch_bounds__(512)                                                                      \
  name(const float* a, const uint8_t* w, float* c, u32 m, u32 n, u32 k, u32 rows_per_wg) {                               \
    extern __shared__ uint8_t few_lds[];                                                                                 \
    const u32 lds_base =                                                                                                 \
        static_cast<u32>(reinterpret_cast<size_t>((const __attribute__((address_space(3))) uint8_t*)few_lds));          \
    const u32 row0 = blockIdx.x * rows_per_wg;                                                                           \
    if (row0 >= n) return;                                                                                               \
    few_i8::q4k_rows<NTOK>(a, w, c, m, n, k, row0, min(rows_per_wg, n - row0), lds_base);                                \
  }
KQ_GEMM_FEW(q4k_gemm_few_t2, 2)
KQ_GEMM_FEW(q4k_gemm_few_t4, 4)

// Legacy "simplified" Q4_K (trueno-gpu/src/kernels/quantize.rs:151-336, kernel name q4k_gemm_fused): blocks of 32
// values in 18 bytes - f16 scale at 0, 16 bytes of nibbles at 2, value i in byte i/2 (low nibble for even i);
// w = scale * q, no min term (:237-267).  W is n rows x k/32 blocks, row-major (:225-231); the product is the
// intended C[m x n] = A[m x k] . W^T, c[row*n + col] (:320-327).  One wave per row of W; lane l takes blocks
// l, l+64, ...; blockIdx.y walks the rows of A.  Blocks are only 2-byte aligned.
// ------------------------------------------------------------------------------------------
extern "C" __global__ void __launch_bounds__(256)
q4k_gemm_fused(const float* a, const uint8_t* b_quant, float* c, u32 m, u32 n, u32 k) {
  const u32 lane = threadIdx.x & 63u, wave = threadIdx.x >> 6, waves = blockDim.x >> 6;
  const u32 nb = k >> 5;
  for (u32 r = blockIdx.y; r < m; r += gridDim.y) {
    const float* ar = a + static_cast<size_t>(r) * k;
    for (u32 col = blockIdx.x * waves + wave; col < n; col += gridDim.x * waves) {
      const uint8_t* rp = b_quant + static_cast<size_t>(col) * nb * 18u;
      float acc = 0.0f;
      for (u32 b = lane; b < nb; b += 64u) {
        const uint8_t* bp = rp + static_cast<size_t>(b) * 18u;
        const float scale = half_bits_to_f32(static_cast<u32>(bp[0]) | (static_cast<u32>(bp[1]) << 8));
        float s = 0.0f;
#pragma unroll
        for (u32 t = 0; t < 16; ++t) {
          const u32 byte = bp[2u + t];
          s = fmaf(static_cast<float>(byte & 15u), ar[32u * b + 2u * t], s);
          s = fmaf(static_cast<float>(byte >> 4), ar[32u * b + 2u * t + 1u], s);
        }
        acc = fmaf(scale, s, acc);
      }
      acc = wave_sum(acc);
      if (lane == 0) c[static_cast<size_t>(r) * n + col] = acc;
    }
  }
}

extern "C" __global__ void __launch_bounds__(256)
q4k_simplified_dequant_f32(float* out, const uint8_t* w, uint64_t n_blocks) {
  const uint64_t stride = static_cast<uint64_t>(gridDim.x) * blockDim.x;
  for (uint64_t gid = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x; gid < n_blocks * 32; gid += stride) {
    const uint8_t* bp = w + (gid >> 5) * 18u;
    const u32 i = static_cast<u32>(gid & 31u);
    const float scale = half_bits_to_f32(static_cast<u32>(bp[0]) | (static_cast<u32>(bp[1]) << 8));
    out[gid] = scale * static_cast<float>((bp[2u + (i >> 1)] >> (4u * (i & 1u))) & 15u);
  }
}

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
    Q::load(r, w + sb * Q::SB, 0u, c);
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

// Read-only yardstick: every wave reads a contiguous run of 1 KB pieces, eight loads in flight per lane, nothing is
// stored.  What a launch over so many bytes costs with no arithmetic: the ceiling the GEMV kernels are compared with.
// Non-temporal loads: every line is asked for once, by one instruction, and then they are the faster ones (258 MB per
// launch: 6.59 TB/s against 5.93 TB/s with ordinary loads, 1.4 GB: 6.9 against 6.15; between four and thirty-two loads
// in flight per lane and between eight and thirty-two waves per CU nothing changes).
extern "C" __global__ void __launch_bounds__(256) kq_read_u128(const u32x4* src, uint64_t n, u32* sink) {
  const u32 lane = threadIdx.x & 63u;
  const uint64_t waves = (static_cast<uint64_t>(gridDim.x) * blockDim.x) >> 6;
  const uint64_t wave = (static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x) >> 6;
  const uint64_t pieces = (n + 63u) / 64u, per_wave = (pieces + waves - 1u) / waves;
  const uint64_t p0 = wave * per_wave, p1 = p0 + per_wave < pieces ? p0 + per_wave : pieces;
  u32 acc = 0u;
  for (uint64_t p = p0; p < p1; p += 8u) {
    u32x4 v[8];
#pragma unroll
    for (int d = 0; d < 8; ++d) {
      const uint64_t i = (p + d) * 64u + lane;
      v[d] = (p + d < p1 && i < n) ? __builtin_nontemporal_load(src + i) : u32x4{0u, 0u, 0u, 0u};
    }
#pragma unroll
    for (int d = 0; d < 8; ++d) acc ^= v[d].x ^ v[d].y ^ v[d].z ^ v[d].w;
  }
  if (acc == 0x9E3779B9u) *sink = acc;
}
