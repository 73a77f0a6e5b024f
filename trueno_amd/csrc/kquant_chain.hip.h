// The GEMV engine of the fast kernels (chain_step) and the resident executor for an ordered list of k-quant
// GEMVs (the weight pass of one decode step).
//
// chain_step computes one workgroup's share of the rows of one matrix: it stages the activation vector in LDS,
// keeps each lane's 64 activations in registers and streams the rows (kquant_quarter.hip.h has the per-row
// arithmetic).  The single-GEMV kernels, the grouped launch and the resident executor all call it, so they give
// the same bits.
//
// Resident executor (phases_body, at the end of this file): the whole list in ONE cooperative launch whose
// workgroups all stay resident.
//   * the host cuts the list into phases of mutually independent entries and deals the workgroups of a phase to
//     its entries in proportion to their bytes;
//   * between phases there is a device-wide barrier: a (two-level) counter in device memory, atomic add to
//     arrive, bounded spin to leave.  A spin that runs out sets a status word and every workgroup exits;
//     nothing can hang;
//   * weights do not depend on activations, so before a workgroup waits at a barrier it has already requested
//     the first rows of its next entry;
//   * the only data that crosses workgroups are the activation vectors and the counters.  The L2s of the eight
//     XCDs are not coherent with each other for ordinary accesses, and the release/acquire fences that would
//     make them so write back / invalidate whole caches (tens of microseconds per barrier, measured).  Instead
//     exactly those accesses are made coherent: y is stored and x is loaded with agent-scope atomic (relaxed)
//     accesses, which go to the memory side; weights are read-only and keep the fast path.
//
// CHAIN_NORM_INPUT: the entry reads x / sqrt(mean(x^2) + 1e-6) instead of x (an RMS normalisation
// without gain, applied as one factor on y; every workgroup stages all of x anyway).  It keeps a
// chain of random matrices in range; the reference has it as a separate kernel
// (trueno-gpu/src/kernels/layernorm.rs:388-470).
#pragma once
#include "kquant_quarter.hip.h"

// One GEMV of a list with the element-wise steps of a decoder layer folded in:
//   x'  = x                         or  silu(x) * x2                         (CHAIN_SWIGLU_INPUT; fused_swiglu)
//   x'' = x' * gamma                (gamma != null)
//   y   = s * (W . x'') + residual  (residual != null),  s = 1 or 1/sqrt(mean(x'^2) + eps)   (CHAIN_NORM_INPUT)
// i.e. rmsnorm(x') * gamma feeds the product (rmsnorm / fused_residual_rmsnorm in front of a projection) and a
// residual add follows it.
struct ChainEntry {
  u32 fmt, k, n, flags;
  const uint8_t* w;
  const float* x;
  float* y;
  const float* gamma;
  const float* x2;
  const float* residual;
  float eps;          // of the normalisation; 0 = kChainNormEps
  u32 pad;
};
enum : u32 { CHAIN_NORM_INPUT = 1u, CHAIN_BARRIER_BEFORE = 2u, CHAIN_SAME_X = 4u, CHAIN_SWIGLU_INPUT = 8u,
             // set by the launcher, never by a caller: the rows of this (one-slab) entry are streamed through LDS
             // (chain_step_stream); the launch's dynamic LDS then includes the waves' rings
             CHAIN_STREAM_LDS = 16u };
constexpr float kChainNormEps = 1e-6f;

// silu(g) * u with the reference's instruction sequence (trueno-gpu/src/kernels/elementwise.rs:565-582)
__device__ __forceinline__ float swiglu1(float g, float u) {
  const float denom = __fadd_rn(1.0f, __builtin_amdgcn_exp2f(__fmul_rn(__fsub_rn(0.0f, g), 1.442695f)));
  return __fmul_rn(__fmul_rn(g, __fdiv_rn(1.0f, denom)), u);
}

// Sum of squares of the activation vector in ONE fixed order, whatever the launch shape: the vector is cut in
// groups of 64 16-byte units (256 values); the sum of a group is the fixed wave butterfly over its units (unit
// 64g + l in lane l, each unit w^2 + (z^2 + (y^2 + x^2)) by FMAs); the groups are added in order.  Any wave can
// take any group, so the sums are formed while the vector is staged and no kernel's result depends on its
// geometry.
__device__ __forceinline__ float unit_sumsq(const f32x4 v) { return fmaf(v.w, v.w, fmaf(v.z, v.z, fmaf(v.y, v.y, v.x * v.x))); }

// the same from a staged copy, by one wave (for engines that stage differently)
template <class Q>
__device__ __forceinline__ float canonical_sumsq_lds(const f32x4* lds4, u32 units, u32 lane) {
  float total = 0.0f;
  for (u32 g = 0; 64u * g < units; ++g) {
    const float sg = wave_sum(unit_sumsq(lds4[Q::swz(64u * g + lane)]));
    total = g == 0u ? sg : total + sg;
  }
  return total;
}

// Barrier counters.  Every workgroup adding to one address costs ~15 ns per add at the memory side
// (8 us for 512 workgroups, measured); arrival is therefore two-level: workgroups arrive at the
// counter of their group of 32, the last one of a group arrives at the top counter, everybody polls
// the top counter (~1.5 us per barrier at 256 workgroups).  One barrier owns kChainBarrierStride
// words: word 0 is the top counter, word 64*(1+g) the counter of group g (each on its own 256 bytes).
constexpr u32 kChainGroup = 32u;
__host__ __device__ constexpr u32 chain_barrier_stride(u32 num_workgroups) {
  return 64u * (1u + (num_workgroups + kChainGroup - 1u) / kChainGroup);
}

__device__ __forceinline__ void chain_arrive(u32* barrier) {
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");     // this thread's coherent y stores have been acknowledged
  __syncthreads();
  if (threadIdx.x == 0) {
    const u32 grp = blockIdx.x / kChainGroup;
    const u32 gsize = min(kChainGroup, gridDim.x - grp * kChainGroup);
    const u32 old = __hip_atomic_fetch_add(barrier + 64u * (1u + grp), 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (old == gsize - 1u) __hip_atomic_fetch_add(barrier, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

// true when every group has arrived; false when the spin budget ran out
__device__ __forceinline__ bool chain_wait(u32* barrier, u32 spin_limit, u32* status, u32* s_flag) {
  if (threadIdx.x == 0) {
    const u32 target = (gridDim.x + kChainGroup - 1u) / kChainGroup;
    u32 spins = 0, ok = 1u;
    while (__hip_atomic_load(barrier, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < target) {
      __builtin_amdgcn_s_sleep(4);
      if (++spins > spin_limit) {
        ok = 0u;
        __hip_atomic_fetch_or(status, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        break;
      }
    }
    *s_flag = ok;
  }
  __syncthreads();
  return *s_flag != 0u;
}

// ------------------------------------------------------------------------------------------------------------
// The engine for matrices of at most 4096 columns (one slab: a wave covers whole rows), weights streamed through LDS.
//
// What the memory system gives a read depends on how it is asked.  Measured on MI355X, 258 MB per launch: the engine's
// own pattern (every lane three 16-byte loads at its quarter of a 144-byte block, so each 128-byte line is asked for by
// three instructions) reads 5.9-6.0 TB/s, and the same with non-temporal loads 4.5 TB/s (a line is fetched again by
// every instruction that asks for a part of it); whole lines asked for once, by non-temporal loads of 1 KB contiguous
// per wave instruction, arrive at 6.55-6.7 TB/s (1.4 GB per launch: 6.9 TB/s against 6.15 TB/s).  So here a batch of U
// rows - U * row bytes, contiguous in memory - is copied to LDS as it lies (global_load_lds_dwordx4, non-temporal, no
// registers held while it is on its way), two batches ahead per wave, and the lanes then read their quarter blocks
// from LDS (Quarter::load_lds: the same pieces as Quarter::load takes from memory).  The arithmetic - and so every bit of
// the result - is chain_step's.
//
// Q4_K and Q5_K rows are whole 16-byte pieces and lie in LDS as in memory; Q6_K blocks (210 bytes, at any even address) are
// re-spaced to 224 bytes by the copy, see below.  Pieces beyond the end of the batch repeat its last piece: a batch is
// always the same number of wave instructions, so the number of copies outstanding is known where the waits are written
// (vmcnt counted by hand; all LDS traffic in asm, see kquant_quarter.hip.h).
//   LDS: [k floats of x, swizzled][rows_per_block partial sums][64 group sums of squares][ring: waves * 2 * slot bytes]
// ------------------------------------------------------------------------------------------------------------
template <int FMT, int U> struct StreamSlot {
  // wave instructions per batch (64 pieces of 16 bytes each): the batch's bytes in LDS, a Q6_K block taking 224
  static constexpr u32 PIECES = (U * 16u * (FMT == FMT_Q6K ? 224u : Quarter<FMT>::SB) + 1023u) / 1024u;
  static constexpr u32 BYTES = PIECES * 1024u;
};

__device__ __forceinline__ u32 lds_addr_of(const void* p) {
  return static_cast<u32>(reinterpret_cast<size_t>((const __attribute__((address_space(3))) uint8_t*)p));
}
__device__ __forceinline__ void dma16_nt(const uint8_t* src, u32 lds_addr) {
  __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                   (__attribute__((address_space(3))) void*)(uintptr_t)lds_addr, 16, 0, 2 /* nt */);
}

template <int FMT, int U>
__device__ __forceinline__ bool chain_step_stream(const ChainEntry& e, f32x4* lds4, u32 row0, u32 rows_per_block, u32 block_threads) {
  using Q = Quarter<FMT>;
  using Slot = StreamSlot<FMT, U>;
  constexpr u32 NL = Slot::PIECES;
  const u32 tid = threadIdx.x, lane = tid & 63u, waves = block_threads >> 6;
  const u32 wave = static_cast<u32>(__builtin_amdgcn_readfirstlane(static_cast<int>(tid >> 6)));
  const u32 k_dim = e.k, n_dim = e.n, nsb = k_dim >> 8;            // 1 <= nsb <= 16
  if (row0 >= n_dim) return true;                                  // the whole workgroup: nothing was touched yet
  const u32 batches = rows_per_block / U;
  const u32 sbl = lane >> 2, c = lane & 3u;
  const u32 row_bytes = nsb * Q::SB;
  const u32 batch_bytes = U * row_bytes;
  const size_t total = static_cast<size_t>(n_dim) * row_bytes;

  const u32 units = k_dim >> 2, xgroups = units >> 6;
  const u32 lds_x = lds_addr_of(lds4);
  const u32 lds_part = lds_x + 16u * units;
  const u32 lds_ss = lds_part + 4u * rows_per_block;
  const u32 lds_ring = ((lds_ss + 256u + 15u) & ~15u) + wave * (2u * Slot::BYTES);
  __shared__ u32 s_next_stream;
  const u32 lds_next = lds_addr_of(&s_next_stream);

  // Batch b of this workgroup into ring slot `slot`; returns the byte shift of the batch inside the slot.
  // Wave instruction j copies the 64 pieces 64 j .. 64 j + 63 of the batch; which bytes of the batch a lane copies with
  // which instruction is the same for every batch, so the offsets are formed once.  Pieces behind the batch's last
  // repeat it, and a batch that does not exist reads the matrix's first batch (from the cache).  A batch that would
  // reach behind the matrix starts as many rows early instead and its rows are found further into the slot.  One form
  // for every case, so that a batch is the same number of copies on every path: a branch between forms is two branches
  // in the assembly, with a path that takes neither as far as a reader of the assembly can tell.
  // Q6_K: a block is 210 bytes, so in a copy of the memory as it lies most blocks would sit at 2-byte alignment in LDS,
  // and a 16-byte LDS read that is not 16-byte aligned takes eight times as long as one that is (27 against 3.4 ns per
  // wave instruction and CU, measured).  So the copy re-spaces the blocks: a lane's 16 bytes may come from any address,
  // and block i of a row goes to 224 i - pieces 0..12 are its bytes 0..207, piece 13 its last 16 bytes (194..209, so d
  // is found at 222 and nothing behind the block is read).  The pieces then come from 2-byte-aligned addresses, which
  // costs the copy (17-22 against 9 ns per wave instruction and CU) far less than it saves the reads.
  constexpr bool kGather = FMT == FMT_Q6K;
  constexpr u32 kPitch = kGather ? 224u : Q::SB;                     // of a block in LDS
  const u32 row_pitch = nsb * kPitch;                                // of a row in LDS
  u32 piece_off[NL];
  if constexpr (!kGather) {
    const u32 last = (batch_bytes - 1u) >> 4;
#pragma unroll
    for (u32 j = 0; j < NL; ++j) {
      const u32 p = 64u * j + lane;
      piece_off[j] = 16u * (p < last ? p : last);
    }
  } else {
    const u32 per_row = 14u * nsb, pieces = U * per_row;
#pragma unroll
    for (u32 j = 0; j < NL; ++j) {
      const u32 p = 64u * j + lane, pc = p < pieces ? p : pieces - 1u;
      const u32 u = pc / per_row, r = pc - u * per_row, blk = r / 14u, jj = r - 14u * blk;
      piece_off[j] = u * row_bytes + blk * Q::SB + (jj < 13u ? 16u * jj : Q::SB - 16u);
    }
  }
  auto issue = [&](u32 b, u32 slot) -> u32 {
    size_t off = static_cast<size_t>(row0 + b * U) * row_bytes;
    const bool exists = b < batches && off < total;
    if (!exists) off = 0;
    const u32 dst = lds_ring + slot * Slot::BYTES;
    u32 shift = 0;
    if (total - off < batch_bytes) {                                  // (total >= batch_bytes: the launcher streams no matrix of fewer than U rows)
      const u32 missing = batch_bytes - static_cast<u32>(total - off);   // whole rows
      shift = kGather ? missing / Q::SB * kPitch : missing;
      off = total - batch_bytes;
    }
    const uint8_t* src = e.w + off;
#pragma unroll
    for (u32 j = 0; j < NL; ++j) dma16_nt(src + piece_off[j], dst + 1024u * j);
    return shift;
  };

  // Activations first (loads return in order, and the vector is an L2 hit), then the first two batches of this wave.
  // The loads of the vector are written in asm like the copies' waits: the compiler, which knows
  // the copies only as memory operations that write LDS, would wait for all of them before it touches LDS at all.
  constexpr u32 kXPre = 4;
  const bool swiglu = (e.flags & CHAIN_SWIGLU_INPUT) != 0u;
  u32x4 xv[kXPre], x2v[kXPre];
#pragma unroll
  for (u32 i = 0; i < kXPre; ++i) {
    const u32 g = wave + i * waves;
    const u32 unit = 64u * (g < xgroups ? g : 0u) + lane;
    asm volatile("global_load_dwordx4 %0, %1, off" : "=&v"(xv[i]) : "v"(reinterpret_cast<const f32x4*>(e.x) + unit) : "memory");
  }
  if (swiglu) {
#pragma unroll
    for (u32 i = 0; i < kXPre; ++i) {
      const u32 g = wave + i * waves;
      const u32 unit = 64u * (g < xgroups ? g : 0u) + lane;
      asm volatile("global_load_dwordx4 %0, %1, off" : "=&v"(x2v[i]) : "v"(reinterpret_cast<const f32x4*>(e.x2) + unit) : "memory");
    }
  }
  u32 cur = wave, nxt = wave + waves;
  bool nxt_in_flight = true;
  const u32 shift_cur0 = issue(cur, 0u), shift_nxt0 = issue(nxt, 1u);      // unconditionally: see issue
  u32 shift_cur = shift_cur0, shift_nxt = shift_nxt0;
  // the vector has landed when only the copies issued behind it are outstanding
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * NL) : "memory");
#pragma unroll
  for (u32 i = 0; i < kXPre; ++i) asm volatile("" : "+v"(xv[i])::"memory");
  if (swiglu) {
#pragma unroll
    for (u32 i = 0; i < kXPre; ++i) asm volatile("" : "+v"(x2v[i]));
  }

  const bool norm = (e.flags & CHAIN_NORM_INPUT) != 0u;
  auto stage = [&](u32 g, f32x4 v) {
    if (norm) {
      const float sg = wave_sum(unit_sumsq(v));
      if (lane == 0) asm volatile("ds_write_b32 %0, %1" ::"v"(lds_ss + 4u * g), "v"(sg) : "memory");
    }
    if (e.gamma) {
      const f32x4 gm = KQ_GLOBAL(f32x4, e.gamma)[64u * g + lane];
      v = f32x4{__fmul_rn(v.x, gm.x), __fmul_rn(v.y, gm.y), __fmul_rn(v.z, gm.z), __fmul_rn(v.w, gm.w)};
    }
    asm volatile("ds_write_b128 %0, %1" ::"v"(lds_x + 16u * Q::swz(64u * g + lane)), "v"(v) : "memory");
  };
  auto as_f32x4 = [](const u32x4& w) { return f32x4{__uint_as_float(w.x), __uint_as_float(w.y), __uint_as_float(w.z), __uint_as_float(w.w)}; };
#pragma unroll
  for (u32 i = 0; i < kXPre; ++i) {
    const u32 g = wave + i * waves;
    if (g < xgroups) {
      f32x4 v = as_f32x4(xv[i]);
      if (swiglu) {
        const f32x4 g2 = as_f32x4(x2v[i]);
        v = f32x4{swiglu1(v.x, g2.x), swiglu1(v.y, g2.y), swiglu1(v.z, g2.z), swiglu1(v.w, g2.w)};
      }
      stage(g, v);
    }
  }
  for (u32 g = wave + kXPre * waves; g < xgroups; g += waves) {     // (workgroups of fewer than four waves)
    f32x4 v = KQ_GLOBAL(f32x4, e.x)[64u * g + lane];
    if (swiglu) {
      const f32x4 g2 = KQ_GLOBAL(f32x4, e.x2)[64u * g + lane];
      v = f32x4{swiglu1(v.x, g2.x), swiglu1(v.y, g2.y), swiglu1(v.z, g2.z), swiglu1(v.w, g2.w)};
    }
    stage(g, v);
  }
  if (tid == 0u) asm volatile("ds_write_b32 %0, %1" ::"v"(lds_next), "v"(2u * waves) : "memory");
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");

  {
    const bool valid = sbl < nsb;
    const u32 sbc = valid ? sbl : nsb - 1u;
    float xr[64];
    float sx[Q::NSUM];
    {
      u32x4 xq[16];
#pragma unroll
      for (int q = 0; q < 16; ++q) {
        const u32 unit = (256u * sbc + Q::value_index(c, 4 * q)) >> 2;
        ldsq_read128<0>(xq[q], lds_x + 16u * Q::swz(unit));
      }
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
      for (int q = 0; q < 16; ++q) asm volatile("" : "+v"(xq[q]));
#pragma unroll
      for (int s = 0; s < Q::NSUM; ++s) sx[s] = 0.0f;
#pragma unroll
      for (int q = 0; q < 16; ++q) {
        f32x4 v = as_f32x4(xq[q]);
        if (!valid) v = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
        xr[4 * q + 0] = v.x; xr[4 * q + 1] = v.y; xr[4 * q + 2] = v.z; xr[4 * q + 3] = v.w;
        sx[Q::sum_index(4 * q)] += (v.x + v.y) + (v.z + v.w);
      }
    }
    typename Q::Regs regs[U];
    for (u32 it = 0; cur < batches; ++it) {
      // batch `cur` has landed when at most the copies of the batch behind it are outstanding
      if (nxt_in_flight) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NL) : "memory");
      else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      const u32 slot = it & 1u;
      const u32 base = lds_ring + slot * Slot::BYTES + shift_cur + sbc * kPitch;
      const u32 rows_here = n_dim - (row0 + cur * U);               // (>= 1) rows behind the matrix's last re-read it: never stored
#pragma unroll
      for (int u = 0; u < U; ++u) Q::load_lds(regs[u], base + (static_cast<u32>(u) < rows_here ? u : rows_here - 1u) * row_pitch, c);
      // the batch after the next: handed out among the waves as they become free (the memory system does not serve
      // them evenly); its copies go where the current batch was, which is in registers when the reads have returned
      u32 nn;
      asm volatile("ds_add_rtn_u32 %0, %1, %2" : "=&v"(nn) : "v"(lds_next), "v"(lane == 0 ? 1u : 0u) : "memory");
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
      for (int u = 0; u < U; ++u) Q::landed(regs[u]);
      asm volatile("" : "+v"(nn));
      nn = static_cast<u32>(__builtin_amdgcn_readfirstlane(static_cast<int>(nn)));
      const bool more = nn < batches;
      u32 shift_nn = 0;
      if (more) shift_nn = issue(nn, slot);
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const float p = wave_sum_lane63(Q::dot(regs[u], c, xr, sx));
        if (lane == 63u) asm volatile("ds_write_b32 %0, %1" ::"v"(lds_part + 4u * (cur * U + u)), "v"(p) : "memory");
      }
      cur = nxt; shift_cur = shift_nxt;
      nxt = nn; shift_nxt = shift_nn;
      nxt_in_flight = more;
    }
  }
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");     // the copies of batches that do not exist; the partial sums
  __syncthreads();
  const float* part = reinterpret_cast<float*>(lds4 + units);
  const float* group_ss = part + rows_per_block;
  float scale = 1.0f;
  if (norm) {
    float total_ss = group_ss[0];
    for (u32 g = 1; g < xgroups; ++g) total_ss += group_ss[g];
    scale = 1.0f / sqrtf(total_ss / static_cast<float>(k_dim) + (e.eps != 0.0f ? e.eps : kChainNormEps));
  }
  for (u32 t = tid; t < rows_per_block; t += block_threads) {
    const u32 row = row0 + t;
    if (row < n_dim) {
      float r = part[t] * scale;
      if (e.residual) r = __fadd_rn(r, KQ_GLOBAL(float, e.residual)[row]);
      KQ_GLOBAL_MUT(float, e.y)[row] = r;
    }
  }
  return true;
}

// One entry on this workgroup's share of rows.  Returns false if the barrier wait gave up.
//   LDS: [k floats of x, swizzled][sw_count * rows_per_block partial sums][k/256 group sums of squares]
// COHERENT: x may have been written, and y may be read, by other workgroups of this same launch.
// block_threads: blockDim.x, handed in by the kernel (an implicit kernel argument, i.e. a load: the kernel decides when).
// chain_step_rows: the workgroup's rows are row0 .. row0 + rows_per_block - 1 (rows_per_block a multiple of U; rows
// beyond the matrix are skipped).  chain_step: block block_id of num_blocks equal blocks of rows.
template <int FMT, int U, bool COHERENT = false>
__device__ __forceinline__ bool chain_step_rows(const ChainEntry& e, u32* wait_counter, u32 spin_limit, u32* status,
                                                f32x4* lds4, u32* s_flag, u32 row0, u32 rows_per_block, u32 block_threads) {
  using Q = Quarter<FMT>;
  // The engine is built for whole waves: a block that is not a positive multiple of 64 threads (the reference's own
  // geometry is 32) would divide by zero below and never leave the staging loop.  Uniform exit before any barrier.
  if (block_threads < 64u || (block_threads & 63u) != 0u) return true;
  if constexpr (!COHERENT)      // (the resident executor keeps the register path: its launcher never sets the flag)
    if ((e.flags & CHAIN_STREAM_LDS) && wait_counter == nullptr) return chain_step_stream<FMT, U>(e, lds4, row0, rows_per_block, block_threads);
  const u32 tid = threadIdx.x, lane = tid & 63u, waves = block_threads >> 6;
  const u32 wave = static_cast<u32>(__builtin_amdgcn_readfirstlane(static_cast<int>(tid >> 6)));   // (the same in every lane: scalar)
  const u32 k_dim = e.k, n_dim = e.n, nsb = k_dim >> 8;
  const u32 slabs = (nsb + 15u) >> 4;
  const u32 sw_count = slabs < waves ? slabs : waves;
  const u32 groups = waves / sw_count;
  const bool has_rows = row0 < n_dim && nsb != 0;
  // Rows go through two sets of registers, one row each: while a row is computed the wave's next row is on its way into
  // the other set.  (Two rows per set and no second set - the same registers - leaves the wave idle while it waits:
  // with three waves to a SIMD the others do not fill that time.  Two sets of two rows do not fit the registers, and a
  // spilled register that is read back inside the loop waits for every load issued before it, the next rows' included.)
  constexpr int UR = 1;
  const u32 batches = has_rows ? rows_per_block / UR : 0u;
  const u32 sw = wave % sw_count, grp = wave / sw_count;
  const bool wave_active = grp < groups && grp < batches;
  const u32 sbl = lane >> 2, c = lane & 3u;
  const size_t row_bytes = static_cast<size_t>(nsb) * Q::SB;
  typename Q::Regs regs[UR], regs_b[UR];
  auto issue = [&](typename Q::Regs (&into)[UR], u32 slab, u32 b) {
    const u32 sb = slab * 16u + sbl;
    const u32 sbc = sb < nsb ? sb : nsb - 1;
#pragma unroll
    for (int u = 0; u < UR; ++u) {
      u32 row = row0 + b * UR + u;
      row = row < n_dim ? row : n_dim - 1;
      Q::load(into[u], e.w + row * row_bytes, sbc * Q::SB, c);     // (a row is tens of KB at most: its vector must fit in LDS)
    }
  };
  // Activations.  Alone on the stream (no barrier to wait for) they are requested BEFORE the weights: loads
  // return in order, so the vector (an L2 hit) is staged and summed while the weights are still on their way.
  // Behind a barrier the weights go first, the vector can only be read once the barrier has opened.
  const u32 units = k_dim >> 2;
  const u32 xgroups = units >> 6;                       // groups of 64 units; k is a multiple of 256
  const f32x4* x4 = reinterpret_cast<const f32x4*>(e.x);
  // Across workgroups of one launch the vector is read past the (per-XCD, mutually incoherent) L2s: 16-byte
  // buffer loads at agent scope (sc1), which the compiler tracks like any other load.
  [[maybe_unused]] __amdgpu_buffer_rsrc_t x_rsrc, x2_rsrc;
  if constexpr (COHERENT) {
    x_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(e.x), 0, static_cast<int>(k_dim * 4u), 0x00020000);
    x2_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(e.x2 ? e.x2 : e.x), 0, static_cast<int>(k_dim * 4u), 0x00020000);
  }
  auto coherent16 = [](__amdgpu_buffer_rsrc_t r, u32 unit) {
    const u32x4 w = __builtin_amdgcn_raw_buffer_load_b128(r, static_cast<int>(16u * unit), 0, 16 /* sc1 */);
    return f32x4{__uint_as_float(w.x), __uint_as_float(w.y), __uint_as_float(w.z), __uint_as_float(w.w)};
  };
  auto load_x = [&](u32 u) {
    f32x4 v;
    if constexpr (COHERENT) v = coherent16(x_rsrc, u);
    else v = KQ_GLOBAL(f32x4, x4)[u];
    if (e.flags & CHAIN_SWIGLU_INPUT) {
      f32x4 g2;
      if constexpr (COHERENT) g2 = coherent16(x2_rsrc, u);
      else g2 = KQ_GLOBAL(f32x4, e.x2)[u];
      v = f32x4{swiglu1(v.x, g2.x), swiglu1(v.y, g2.y), swiglu1(v.z, g2.z), swiglu1(v.w, g2.w)};
    }
    return v;
  };
  constexpr u32 kXPre = 4;                              // groups per wave requested ahead of the weights
  f32x4 xv[kXPre];
  const bool x_first = wait_counter == nullptr && has_rows;
  if (x_first) {
#pragma unroll
    for (u32 i = 0; i < kXPre; ++i) {
      const u32 g = wave + i * waves;
      xv[i] = load_x(64u * (g < xgroups ? g : 0u) + lane);
    }
  }
  // in flight across the barrier and the activation staging.  Issued by every wave, also one without rows
  // (it reads clamped, valid addresses and ignores them): a branch here would hide the number of loads in
  // flight from the compiler, which then waits for all of them before the first activation is staged.
  // The wave that polls a barrier asks for its rows only when the barrier has opened: loads return in order, and the
  // answer to a poll behind weight loads comes late, for the whole workgroup.
  const bool polls = wait_counter != nullptr && wave == 0u;
  if (!polls) issue(regs, sw, wave_active ? grp : 0u);        // the host never launches this engine with k = 0 or n = 0

  if (wait_counter && !chain_wait(wait_counter, spin_limit, status, s_flag)) return false;
  if (polls) issue(regs, sw, wave_active ? grp : 0u);
  if (!has_rows) return true;

  float* part = reinterpret_cast<float*>(lds4 + units);
  float* group_ss = part + sw_count * rows_per_block;   // one sum of squares per group of 64 units
  const bool norm = (e.flags & CHAIN_NORM_INPUT) != 0u;
  auto stage = [&](u32 g, f32x4 v) {
    if (norm) {
      const float sg = wave_sum(unit_sumsq(v));
      if (lane == 0) group_ss[g] = sg;
    }
    if (e.gamma) {                      // weights of the normalisation, never written inside a launch
      const f32x4 gm = KQ_GLOBAL(f32x4, e.gamma)[64u * g + lane];
      v = f32x4{__fmul_rn(v.x, gm.x), __fmul_rn(v.y, gm.y), __fmul_rn(v.z, gm.z), __fmul_rn(v.w, gm.w)};
    }
    lds4[Q::swz(64u * g + lane)] = v;
  };
  if (x_first) {
#pragma unroll
    for (u32 i = 0; i < kXPre; ++i) {
      const u32 g = wave + i * waves;
      if (g < xgroups) stage(g, xv[i]);
    }
  }
  for (u32 g = wave + (x_first ? kXPre * waves : 0u); g < xgroups; g += waves) stage(g, load_x(64u * g + lane));
  // Workgroup barrier over the LDS writes only.  __syncthreads() would also drain the weight loads that are in
  // flight (the compiler waits for every outstanding memory operation before s_barrier), which is the one thing
  // the ordering above is there to avoid.
  // Batches of rows after a wave's first are handed out as waves become free (one counter per slab index, so
  // that the waves sharing a row's slabs each see every batch once): the memory system does not serve the waves
  // evenly, and the workgroup is only done when its slowest wave is.
  __shared__ u32 s_next[16];
  if (tid < 16u) s_next[tid] = groups;
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
  float scale = 1.0f;
  if (norm) {
    float total = group_ss[0];
    for (u32 g = 1; g < xgroups; ++g) total += group_ss[g];
    scale = 1.0f / sqrtf(total / static_cast<float>(k_dim) + (e.eps != 0.0f ? e.eps : kChainNormEps));
  }

  if (wave_active) {
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
      const bool handed_out = slabs <= waves && waves >= 8u;   // every wave owns one slab; small workgroups gain nothing
      // the row after b for this wave (handed out as waves become free, or every groups-th one)
      auto next_of = [&](u32 b) -> u32 {
        if (!handed_out) return b + groups;
        u32 nb = 0u;
        if (lane == 0) nb = __hip_atomic_fetch_add(&s_next[sw], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        return static_cast<u32>(__builtin_amdgcn_readfirstlane(static_cast<int>(nb)));
      };
      // One step: the wave's next row is asked for into `nxt`, then row b (in `cur`) is computed.  The next row is asked
      // for always: when there is none it is the last row once more (from the cache, ignored) - a branch around the
      // loads would hide from the compiler how many are in flight where it places the wait for this row's.
      auto step = [&](typename Q::Regs (&cur)[UR], typename Q::Regs (&nxt)[UR], u32 b) -> u32 {
        const u32 nb = next_of(b);
        issue(nxt, slab, nb < batches ? nb : batches - 1u);
        __builtin_amdgcn_sched_barrier(0);      // (the loads stay in front of the arithmetic whatever the register pressure)
#pragma unroll
        for (int u = 0; u < UR; ++u) {
          const float p = wave_sum_lane63(Q::dot(cur[u], c, xr, sx));
          if (lane == 63u) {
            const u32 idx = sw * rows_per_block + b * UR + u;
            part[idx] = (slab == sw) ? p : part[idx] + p;
          }
        }
        return nb;
      };
      u32 b = grp;
      if (slab != sw) issue(regs, slab, b);
      while (true) {
        b = step(regs, regs_b, b);
        if (b >= batches) break;
        b = step(regs_b, regs, b);
        if (b >= batches) break;
      }
    }
  }
  __syncthreads();
  for (u32 t = tid; t < rows_per_block; t += block_threads) {
    const u32 row = row0 + t;
    if (row < n_dim) {
      float s = part[t];
      for (u32 i = 1; i < sw_count; ++i) s += part[i * rows_per_block + t];
      float r = s * scale;
      if constexpr (COHERENT) {
        if (e.residual)
          r = __fadd_rn(r, __uint_as_float(__hip_atomic_load(KQ_GLOBAL(u32, e.residual) + row, __ATOMIC_RELAXED,
                                                             __HIP_MEMORY_SCOPE_AGENT)));
        __hip_atomic_store(KQ_GLOBAL_MUT(u32, e.y) + row, __float_as_uint(r), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      } else {
        if (e.residual) r = __fadd_rn(r, KQ_GLOBAL(float, e.residual)[row]);
        KQ_GLOBAL_MUT(float, e.y)[row] = r;
      }
    }
  }
  return true;
}

template <int FMT, int U, bool COHERENT = false>
__device__ __forceinline__ bool chain_step(const ChainEntry& e, u32* wait_counter, u32 spin_limit, u32* status,
                                           f32x4* lds4, u32* s_flag, u32 block_id, u32 num_blocks, u32 block_threads) {
  u32 rows_per_block = (e.n + num_blocks - 1) / num_blocks;
  rows_per_block = ((rows_per_block + U - 1) / U) * U;
  return chain_step_rows<FMT, U, COHERENT>(e, wait_counter, spin_limit, status, lds4, s_flag, block_id * rows_per_block, rows_per_block,
                                           block_threads);
}

// ------------------------------------------------------------------------------------------------------------
// Phase executor: the whole list in one resident launch of ONE workgroup per CU.  The host cuts the list into
// phases of mutually independent entries and, per phase, deals the workgroups to the entries in proportion to
// their bytes (PhaseAssign, one per phase and workgroup).  A workgroup computes its share of its entry exactly
// as a separate launch would, with a device-wide barrier between phases.  The loop over phases is written per
// format (a workgroup stays in one format's loop for as long as its assignments keep that format): with the
// three engines side by side in one loop body the register allocator needs half again as many registers.
// ------------------------------------------------------------------------------------------------------------
struct PhaseAssign {
  u32 entry;        // index into the entry list
  u32 block_id;     // this workgroup's index among the num_blocks workgroups of that entry
  u32 num_blocks;
  u32 fmt;          // format of that entry; 0 = this workgroup has nothing to do in this phase
};

template <int FMT, int U>
__device__ __forceinline__ u32 phases_run(u32 p, const ChainEntry* __restrict__ entries, const PhaseAssign* __restrict__ assign,
                                          u32 phases, u32* counters, u32* status, u32 spin_limit, f32x4* lds4, u32* s_flag) {
  const u32 stride = chain_barrier_stride(gridDim.x);
  for (; p < phases; ++p) {
    const PhaseAssign a = assign[static_cast<size_t>(p) * gridDim.x + blockIdx.x];
    if (a.fmt != static_cast<u32>(FMT)) break;
    const ChainEntry e = entries[a.entry];
    if (!chain_step<FMT, U, true>(e, p ? counters + p * stride : nullptr, spin_limit, status, lds4, s_flag, a.block_id, a.num_blocks, blockDim.x))
      return 0xFFFFFFFFu;
    if (p + 1 < phases) chain_arrive(counters + (p + 1) * stride);
    else __syncthreads();
  }
  return p;
}

template <int U>
__device__ __forceinline__ void phases_body(const ChainEntry* __restrict__ entries, const PhaseAssign* __restrict__ assign,
                                            u32 phases, u32* counters, u32* status, u32 spin_limit) {
  extern __shared__ f32x4 lds4[];
  __shared__ u32 s_flag;
  const u32 stride = chain_barrier_stride(gridDim.x);
  u32 p = 0;
  while (p < phases) {
    const u32 fmt = assign[static_cast<size_t>(p) * gridDim.x + blockIdx.x].fmt;
    if (fmt == FMT_Q4K) p = phases_run<FMT_Q4K, U>(p, entries, assign, phases, counters, status, spin_limit, lds4, &s_flag);
    else if (fmt == FMT_Q5K) p = phases_run<FMT_Q5K, U>(p, entries, assign, phases, counters, status, spin_limit, lds4, &s_flag);
    else if (fmt == FMT_Q6K) p = phases_run<FMT_Q6K, U>(p, entries, assign, phases, counters, status, spin_limit, lds4, &s_flag);
    else {                                   // idle in this phase: keep the barriers in step
      if (p && !chain_wait(counters + p * stride, spin_limit, status, &s_flag)) return;
      if (p + 1 < phases) chain_arrive(counters + (p + 1) * stride);
      ++p;
    }
  }
}
