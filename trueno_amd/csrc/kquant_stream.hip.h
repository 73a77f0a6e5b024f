// Streaming executor for an ordered list of k-quant GEMVs: the weight pass of a decode step as ONE
// launch in which HBM never waits for compute, barriers or activations.
//
// One workgroup per CU, resident for the whole list.  Wave 0 is the PRODUCER: it walks the list and
// copies this workgroup's share of every matrix - a contiguous run of rows, hence a contiguous run
// of bytes - from HBM into a ring buffer in LDS with direct-to-LDS loads (global_load_lds_dwordx4,
// 64 lanes x 16 bytes = 1 KB per instruction, no registers in between), up to ~56 KB in flight and up
// to a whole ring ahead of the consumers.  Weights do not depend on activations, so the producer
// runs straight through device-wide barriers.  The other waves are CONSUMERS: they take rows out of
// the ring (quarter-block engine of kquant_quarter.hip.h, activations in registers), and at a
// dependency they arrive at / wait for the device-wide barrier and stage the new activation vector.
//
// Flow control is two monotonic counters in LDS, in KB of stream: `filled` (producer: everything
// below has landed) and one `done` word per consumer wave (nothing below is needed any more).  The
// producer publishes what has landed after each packet (s_waitcnt vmcnt(N) bounds what is still in
// flight), and before it ever sleeps for space it first drains and publishes everything it has
// requested, so no consumer can wait for bytes whose publication waits for that consumer.
// The ring is a byte FIFO: row r of entry e sits at stream offset S_e + r*row_bytes (mod ring size);
// the 16 bytes after the ring mirror its first 16, so a 16-byte read may straddle the wrap.
//
// Consumers never meet the producer at a barrier: they synchronise among themselves with a counter
// barrier in LDS.  Where several waves share a row (K > 4096: one wave per slab of 16 super-blocks)
// the partial sums meet in LDS and the last wave to arrive adds them in slab order, so results do
// not depend on timing.  Every wait in this file is bounded: a wait that runs out raises the
// workgroup's abort flag and the status word, and every wave leaves.
//
// Cross-workgroup data (x, y, barrier counters) is accessed with agent-scope atomics (coherent
// across XCDs); weights are read-only.
#pragma once
#include "kquant_chain.hip.h"

#ifdef STREAM_TS
// debug timeline: [entry][8] = consumer0: enter, staged, rows done, (spare); producer: start, end, blocked ticks, (spare)
extern __device__ unsigned long long* g_stream_ts;
extern __device__ unsigned g_stream_ts_wg;
#define STREAM_STAMP(entry, slot) do { if (g_stream_ts && blockIdx.x == g_stream_ts_wg && (threadIdx.x & 63u) == 0u) g_stream_ts[8 * (entry) + (slot)] = wall_clock64(); } while (0)
#define STREAM_ADD(entry, slot, v) do { if (g_stream_ts && blockIdx.x == g_stream_ts_wg && (threadIdx.x & 63u) == 0u) g_stream_ts[8 * (entry) + (slot)] += (v); } while (0)
#else
#define STREAM_STAMP(entry, slot) do { } while (0)
#define STREAM_ADD(entry, slot, v) do { } while (0)
#endif

namespace stream {

constexpr u32 kRingKB = 96;
constexpr u32 kRingBytes = kRingKB * 1024u;
constexpr u32 kPacketKB = 8;            // DMA instructions issued between two flow-control checks
constexpr u32 kInFlightKB = 48;         // s_waitcnt vmcnt(48): at most this many KB not yet landed after a publish
constexpr u32 kMaxConsumers = 12;
constexpr u32 kLocalSpinLimit = 40000000u;   // polls of an LDS word (each ~0.1 us): seconds

typedef __attribute__((address_space(3))) uint8_t* lds_bytes;

// LDS words are polled and published through inline asm so the compiler does not order them against
// (i.e. drain) the direct-to-LDS loads in flight.
__device__ __forceinline__ u32 lds_ld(u32 addr) {
  u32 v;
  asm volatile("ds_read_b32 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(v) : "v"(addr) : "memory");
  return v;
}
__device__ __forceinline__ void lds_st(u32 addr, u32 v) { asm volatile("ds_write_b32 %0, %1" ::"v"(addr), "v"(v) : "memory"); }
__device__ __forceinline__ u32 lds_add_rtn(u32 addr, u32 v) {
  u32 old;
  asm volatile("ds_add_rtn_u32 %0, %1, %2\n\ts_waitcnt lgkmcnt(0)" : "=v"(old) : "v"(addr), "v"(v) : "memory");
  return old;
}
// A read's result register is only defined once the wait inside the same asm statement has passed;
// nothing asynchronous is ever left pending across statements.
__device__ __forceinline__ u32x4 lds_ld128(u32 addr) {
  u32x4 v;
  asm volatile("ds_read_b128 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(v) : "v"(addr) : "memory");
  return v;
}
__device__ __forceinline__ void lds_ld128x3(u32x4& a, u32x4& b, u32x4& c, u32 aa, u32 ab, u32 ac) {
  asm volatile("ds_read_b128 %0, %3\n\tds_read_b128 %1, %4\n\tds_read_b128 %2, %5\n\ts_waitcnt lgkmcnt(0)"
               : "=&v"(a), "=&v"(b), "=&v"(c) : "v"(aa), "v"(ab), "v"(ac) : "memory");
}
__device__ __forceinline__ u32x2 lds_ld64(u32 addr) {
  u32x2 v;
  asm volatile("ds_read_b64 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(v) : "v"(addr) : "memory");
  return v;
}
__device__ __forceinline__ u32 lds_ld16(u32 addr) {
  u32 v;
  asm volatile("ds_read_u16 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(v) : "v"(addr) : "memory");
  return v;
}
__device__ __forceinline__ void lds_wait() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }

// control block at the start of dynamic LDS (byte offsets)
enum : u32 {
  kCtlFilled = 0, kCtlAbort = 4, kCtlBarCount = 8, kCtlBarGen = 12, kCtlGate = 16,
  kCtlDone = 64,                      // kMaxConsumers words
  kCtlRed = 128,                      // 16 floats
  kCtlBytes = 256
};

struct Layout {   // byte offsets in dynamic LDS
  u32 ring, x, part, cnt;
};
__host__ __device__ inline Layout layout(u32 x_bytes_max, u32 rows_max, u32 slabs_max) {
  Layout l;
  l.ring = kCtlBytes;
  l.x = l.ring + kRingBytes + 16u;
  l.part = l.x + x_bytes_max;
  l.cnt = l.part + rows_max * slabs_max * 4u;
  return l;
}
__host__ __device__ inline u32 lds_bytes_needed(u32 x_bytes_max, u32 rows_max, u32 slabs_max) {
  return layout(x_bytes_max, rows_max, slabs_max).cnt + rows_max * 4u;
}

struct Share {    // this workgroup's share of one entry
  u32 row0, rows, nsb, sb_bytes;
  size_t row_bytes;
  u32 bytes, chunks;                  // bytes of the share and KB of ring it takes
};
__device__ __forceinline__ Share share_of(const ChainEntry& e) {
  Share s;
  s.nsb = e.k >> 8;
  s.sb_bytes = e.fmt == FMT_Q4K ? 144u : e.fmt == FMT_Q5K ? 176u : 210u;
  s.row_bytes = static_cast<size_t>(s.nsb) * s.sb_bytes;
  const u32 per = (e.n + gridDim.x - 1) / gridDim.x;
  s.row0 = blockIdx.x * per;
  s.rows = s.row0 < e.n ? min(per, e.n - s.row0) : 0u;
  s.bytes = s.rows * static_cast<u32>(s.row_bytes);
  s.chunks = (s.bytes + 1023u) >> 10;
  return s;
}

__device__ __forceinline__ u32 wrap(u32 off) { return off >= kRingBytes ? off - kRingBytes : off; }

// ---- producer --------------------------------------------------------------------------------------
__device__ __forceinline__ void producer(const ChainEntry* __restrict__ entries, u32 count, u32 consumers,
                                         u32 lds_base, u32* status) {
  const u32 lane = threadIdx.x & 63u;
  const u32 a_filled = lds_base + kCtlFilled, a_abort = lds_base + kCtlAbort, a_done = lds_base + kCtlDone;
  const u32 ring = lds_base + layout(0, 0, 0).ring;
  u32 issued = 0;        // KB of stream requested so far
  u32 published = 0;
  u32 free_below = 0;    // min over consumers of their `done` word, as last read
  auto publish = [&](u32 upto) {
    if (upto <= published) return;
    // the chunk at ring offset 0 is mirrored behind the ring before it becomes visible
    const u32 first_lap = (published + kRingKB - 1) / kRingKB, last_lap = (upto - 1) / kRingKB;
    if (first_lap <= last_lap && first_lap * kRingKB < upto) {
      if (lane == 0) {
        const u32x4 v = lds_ld128(ring);
        asm volatile("ds_write_b128 %0, %1" ::"v"(ring + kRingBytes), "v"(v) : "memory");
      }
    }
    lds_st(a_filled, upto);
    published = upto;
  };
  for (u32 i = 0; i < count; ++i) {
    const ChainEntry e = entries[i];
    const Share s = share_of(e);
    STREAM_STAMP(i, 4);
    const uint8_t* base = e.w + static_cast<size_t>(s.row0) * s.row_bytes;
    const u32 last_piece = s.bytes >= 16u ? ((s.bytes - 1u) & ~15u) : 0u;   // offset of the last 16-byte piece
    for (u32 c = 0; c < s.chunks; c += kPacketKB) {
      const u32 pk = min(kPacketKB, s.chunks - c);
      if (issued + pk > free_below + kRingKB) {
        __builtin_amdgcn_s_waitcnt(0x0F70);          // vmcnt(0): everything requested has landed
        publish(issued);
#ifdef STREAM_TS
        const unsigned long long tb0 = wall_clock64();
#endif
        u32 spins = 0;
        for (;;) {
          u32 mn = lds_ld(a_done);
          for (u32 w = 1; w < consumers; ++w) mn = min(mn, lds_ld(a_done + 4u * w));
          free_below = mn;
          if (issued + pk <= free_below + kRingKB) {
#ifdef STREAM_TS
            STREAM_ADD(i, 6, wall_clock64() - tb0);
#endif
            break;
          }
          if (lds_ld(a_abort) != 0u) return;
          if (++spins > kLocalSpinLimit) {
            lds_st(a_abort, 1u);
            if (lane == 0) __hip_atomic_fetch_or(status, 2u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
            return;
          }
          __builtin_amdgcn_s_sleep(2);
        }
      }
      for (u32 j = 0; j < pk; ++j) {
        const u32 off = min(((c + j) << 10) + lane * 16u, last_piece);
        const u32 slot = (issued + j) % kRingKB;
        __builtin_amdgcn_global_load_lds(
            (const __attribute__((address_space(1))) void*)(base + off),
            (__attribute__((address_space(3))) void*)(uintptr_t)(ring + (slot << 10)), 16, 0, 0);
      }
      issued += pk;
      if (issued > kInFlightKB) {
        __builtin_amdgcn_s_waitcnt(0x0F70 | (kInFlightKB & 15u) | ((kInFlightKB >> 4) << 14));
        publish(issued - kInFlightKB);
      }
    }
    STREAM_STAMP(i, 5);
  }
  __builtin_amdgcn_s_waitcnt(0x0F70);
  publish(issued);
}

// ---- consumer-side synchronisation ---------------------------------------------------------------
// Counter barrier among the consumer waves.  Returns false on abort.
__device__ __forceinline__ bool consumer_barrier(u32 lds_base, u32 consumers, u32& gen, u32* status) {
  const u32 lane = threadIdx.x & 63u;
  u32 ok = 1u;
  ++gen;
  if (lane == 0) {
    const u32 old = lds_add_rtn(lds_base + kCtlBarCount, 1u);
    if (old == consumers - 1u) {
      lds_st(lds_base + kCtlBarCount, 0u);
      lds_st(lds_base + kCtlBarGen, gen);
    } else {
      u32 spins = 0;
      while (lds_ld(lds_base + kCtlBarGen) != gen) {
        if (lds_ld(lds_base + kCtlAbort) != 0u) { ok = 0u; break; }
        if (++spins > kLocalSpinLimit) {
          lds_st(lds_base + kCtlAbort, 1u);
          __hip_atomic_fetch_or(status, 4u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
          ok = 0u;
          break;
        }
        __builtin_amdgcn_s_sleep(1);
      }
    }
  }
  ok = static_cast<u32>(__builtin_amdgcn_readfirstlane(static_cast<int>(ok)));
  return ok != 0u;
}

// quarter-block registers out of the ring: the same bytes Quarter<FMT>::load takes from global memory
template <int FMT>
__device__ __forceinline__ void load_from_ring(typename Quarter<FMT>::Regs& r, u32 ring, u32 off, u32 c) {
  if constexpr (FMT == FMT_Q4K) {
    lds_ld128x3(r.hdr, r.q0, r.q1, ring + wrap(off), ring + wrap(off + 16u + 32u * c), ring + wrap(off + 32u + 32u * c));
  } else if constexpr (FMT == FMT_Q5K) {
    u32x4 h;
    lds_ld128x3(h, r.q0, r.q1, ring + wrap(off), ring + wrap(off + 16u + 32u * c), ring + wrap(off + 32u + 32u * c));
    r.qh = lds_ld64(ring + wrap(off + 144u + 8u * c));
    r.dd = h.x;
    // the 24 bits at byte 4 + 3c of the block
    const u32 f1 = __builtin_amdgcn_alignbit(h.z, h.y, 24), f2 = __builtin_amdgcn_alignbit(h.w, h.z, 16), f3 = h.w >> 8;
    r.f24 = c == 0u ? h.y : c == 1u ? f1 : c == 2u ? f2 : f3;
  } else {
    const u32 h = c >> 1, is = c & 1u;
    lds_ld128x3(r.a, r.b, r.c, ring + wrap(off + 64u * h + 16u * is), ring + wrap(off + 64u * h + 32u + 16u * is),
                ring + wrap(off + 128u + 32u * h + 16u * is));
    r.sc = lds_ld64(ring + wrap(off + 192u + 8u * h));
    r.d = lds_ld16(ring + wrap(off + 208u));
  }
}

struct ConsumerState {
  u32 lds_base, ring, consumers, me;   // me: consumer index 0..consumers-1
  u32 bar_gen;
  u32 stream_kb;                       // stream position (KB) where the current entry starts
  u32 filled_seen;
  u32* status;
  u32 spin_limit;
  u32 entry_index;
  float norm_scale;                    // 1/sqrt(mean(x^2)+eps) of the vector staged in LDS
  const float* xr_x;                   // which activation vector / length / swizzle class the registers hold
  u32 xr_k, xr_class;
};

__device__ __forceinline__ bool wait_filled(ConsumerState& st, u32 need_kb) {
  if (st.filled_seen >= need_kb) return true;
  u32 spins = 0;
  for (;;) {
    st.filled_seen = lds_ld(st.lds_base + kCtlFilled);
    if (st.filled_seen >= need_kb) return true;
    if (lds_ld(st.lds_base + kCtlAbort) != 0u) return false;
    if (++spins > kLocalSpinLimit) {
      lds_st(st.lds_base + kCtlAbort, 1u);
      if ((threadIdx.x & 63u) == 0u) __hip_atomic_fetch_or(st.status, 8u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
      return false;
    }
    __builtin_amdgcn_s_sleep(1);
  }
}

// One entry, consumer side.  xr/sx persist across entries that read the same activation vector.
template <int FMT>
__device__ __forceinline__ bool consume_entry(ConsumerState& st, const ChainEntry& e, const Layout& lay, u32* barrier_arrive,
                                              u32* barrier_wait, bool same_x, float (&xr)[64],
                                              float (&sx)[Quarter<FMT>::NSUM], float& scale) {
  using Q = Quarter<FMT>;
  const u32 lane = threadIdx.x & 63u;
  const Share s = share_of(e);
  const u32 slabs = (s.nsb + 15u) >> 4;
  const u32 sw_count = min(slabs, st.consumers);
  const u32 groups = st.consumers / sw_count;
  const u32 grp = st.me / sw_count, sw = st.me % sw_count;
  const bool wave_active = grp < groups && s.rows != 0u;
  const u32 next_kb = st.stream_kb + s.chunks;
  const u32 a_done = st.lds_base + kCtlDone + 4u * st.me;
  const u32 ctid = threadIdx.x - 64u, cthreads = st.consumers * 64u;   // thread index among the consumers
  if (st.me == 0u) STREAM_STAMP(st.entry_index, 0);

  if (!same_x) {
    // everybody is done with the previous activations (and, before a device barrier, with its rows)
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if (!consumer_barrier(st.lds_base, st.consumers, st.bar_gen, st.status)) return false;
    if (st.me == 0u) STREAM_STAMP(st.entry_index, 3);
    if (barrier_arrive || barrier_wait) {
      if (st.me == 0u) {
        u32 ok = 1u;
        if (lane == 0u) {
          if (barrier_arrive) {
            const u32 g = blockIdx.x / kChainGroup, gsize = min(kChainGroup, gridDim.x - g * kChainGroup);
            const u32 old = __hip_atomic_fetch_add(barrier_arrive + 64u * (1u + g), 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (old == gsize - 1u) __hip_atomic_fetch_add(barrier_arrive, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          }
          if (barrier_wait) {
            const u32 target = (gridDim.x + kChainGroup - 1u) / kChainGroup;
            u32 spins = 0;
            while (__hip_atomic_load(barrier_wait, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < target) {
              __builtin_amdgcn_s_sleep(4);
              if (++spins > st.spin_limit || lds_ld(st.lds_base + kCtlAbort) != 0u) {
                ok = 0u;
                lds_st(st.lds_base + kCtlAbort, 1u);
                __hip_atomic_fetch_or(st.status, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
                break;
              }
            }
          }
        }
        (void)ok;
      }
      if (!consumer_barrier(st.lds_base, st.consumers, st.bar_gen, st.status)) return false;
      if (lds_ld(st.lds_base + kCtlAbort) != 0u) return false;
    }
    if (st.me == 0u) STREAM_STAMP(st.entry_index, 7);
    // stage the activation vector (coherent loads), swizzled for this format's register slices
    const u32 units = e.k >> 2;
    const u32 x_lds = st.lds_base + lay.x;
    // the vector was written by other workgroups of this launch: 16-byte buffer loads at agent scope (sc1)
    const __amdgpu_buffer_rsrc_t x_rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(e.x), 0, static_cast<int>(e.k * 4u), 0x00020000);
    for (u32 u = ctid; u < units; u += cthreads) {
      const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(x_rsrc, static_cast<int>(16u * u), 0, 16);
      asm volatile("ds_write_b128 %0, %1" ::"v"(x_lds + 16u * Q::swz(u)), "v"(v) : "memory");
    }
    lds_wait();
    if (!consumer_barrier(st.lds_base, st.consumers, st.bar_gen, st.status)) return false;
    if (st.me == 0u) STREAM_STAMP(st.entry_index, 2);
    // sum of squares in the fixed order of kquant_chain.hip.h (groups of 64 units), per wave
    float ss = 0.0f;
    for (u32 g = 0; 64u * g < units; ++g) {
      const u32x4 v = lds_ld128(x_lds + 16u * Q::swz(64u * g + lane));
      const f32x4 f = {__uint_as_float(v.x), __uint_as_float(v.y), __uint_as_float(v.z), __uint_as_float(v.w)};
      const float sg = wave_sum(unit_sumsq(f));
      ss = g == 0u ? sg : ss + sg;
    }
    st.norm_scale = 1.0f / sqrtf(ss / static_cast<float>(e.k) + kChainNormEps);
  } else {
    // rows shared by several waves reuse the partial-sum slots of the previous entry: everybody must be
    // through with them
    if (slabs > 1u && !consumer_barrier(st.lds_base, st.consumers, st.bar_gen, st.status)) return false;
  }
  scale = (e.flags & CHAIN_NORM_INPUT) ? st.norm_scale : 1.0f;
  if (st.me == 0u) STREAM_STAMP(st.entry_index, 1);

  if (!wave_active) {
    lds_st(a_done, next_kb);
    st.stream_kb = next_kb;
    return true;
  }
  const u32 sbl = lane >> 2, c = lane & 3u;
  const u32 part = st.lds_base + lay.part, cnt = st.lds_base + lay.cnt;
  const u32 entry_off = (st.stream_kb % kRingKB) << 10;    // ring offset of the share's first byte
  for (u32 slab = sw; slab < slabs; slab += sw_count) {
    const u32 sb = slab * 16u + sbl;
    const bool valid = sb < s.nsb;
    const u32 sbc = valid ? sb : s.nsb - 1u;
    const u32 cls = FMT == FMT_Q6K ? 1u : 0u;
    if (!same_x || slabs > sw_count || st.xr_x != e.x || st.xr_k != e.k || st.xr_class != cls) {
      st.xr_x = e.x;
      st.xr_k = e.k;
      st.xr_class = cls;
      // this wave's register slice of the activations for the slab
#pragma unroll
      for (int t = 0; t < Q::NSUM; ++t) sx[t] = 0.0f;
#pragma unroll
      for (int q = 0; q < 16; ++q) {
        const u32 unit = (256u * sbc + Q::value_index(c, 4 * q)) >> 2;
        u32x4 v = lds_ld128(st.lds_base + lay.x + 16u * Q::swz(unit));
        if (!valid) v = u32x4{0u, 0u, 0u, 0u};
        xr[4 * q + 0] = __uint_as_float(v.x); xr[4 * q + 1] = __uint_as_float(v.y);
        xr[4 * q + 2] = __uint_as_float(v.z); xr[4 * q + 3] = __uint_as_float(v.w);
        sx[Q::sum_index(4 * q)] += (xr[4 * q] + xr[4 * q + 1]) + (xr[4 * q + 2] + xr[4 * q + 3]);
      }
    }
    for (u32 r = grp; r < s.rows; r += groups) {
      const u32 row_off = r * static_cast<u32>(s.row_bytes);
      const u32 need_kb = st.stream_kb + min(s.chunks, (row_off + static_cast<u32>(s.row_bytes) + 16u + 1023u) >> 10);
      if (!wait_filled(st, need_kb)) return false;
      typename Q::Regs regs;
      load_from_ring<FMT>(regs, st.ring, (entry_off + row_off + sbc * Q::SB) % kRingBytes, c);
      const float p = wave_sum(Q::dot(regs, c, xr, sx));
      if (slabs == 1u) {
        if (lane == 0u)
          __hip_atomic_store(reinterpret_cast<u32*>(e.y) + s.row0 + r, __float_as_uint(p * scale), __ATOMIC_RELAXED,
                             __HIP_MEMORY_SCOPE_AGENT);
      } else if (lane == 0u) {
        // partial sums meet in LDS; the last slab to arrive adds them in slab order
        const u32 slot = part + 4u * (r * slabs + slab);
        lds_st(slot, __float_as_uint(p));
        lds_wait();
        const u32 old = lds_add_rtn(cnt + 4u * r, 1u);
        if (old == slabs - 1u) {
          float tot = 0.0f;
          for (u32 t = 0; t < slabs; ++t) tot += __uint_as_float(lds_ld(part + 4u * (r * slabs + t)));
          lds_st(cnt + 4u * r, 0u);
          __hip_atomic_store(reinterpret_cast<u32*>(e.y) + s.row0 + r, __float_as_uint(tot * scale), __ATOMIC_RELAXED,
                             __HIP_MEMORY_SCOPE_AGENT);
        }
      }
      // nothing below the next row this wave will read is needed any more (last slab pass only)
      if (slab + sw_count >= slabs) {
        const u32 nr = r + groups;
        lds_st(a_done, nr < s.rows ? st.stream_kb + ((nr * static_cast<u32>(s.row_bytes)) >> 10) : next_kb);
      }
    }
  }
  lds_st(a_done, next_kb);
  st.stream_kb = next_kb;
  return true;
}

// The whole list.  Block = 64 * (1 + consumers) threads, grid = one workgroup per CU (cooperative launch).
__device__ __forceinline__ void stream_body(const ChainEntry* __restrict__ entries, u32 count, u32* counters, u32* status,
                                            u32 spin_limit, u32 x_bytes_max, u32 rows_max, u32 slabs_max) {
  extern __shared__ f32x4 lds4[];
  const u32 lds_base = (u32)(uintptr_t)(lds_bytes)lds4;   // LDS address of the dynamic segment
  const u32 tid = threadIdx.x, wave = tid >> 6, consumers = (blockDim.x >> 6) - 1u;
  const Layout lay = layout(x_bytes_max, rows_max, slabs_max);
  u32* ctl = reinterpret_cast<u32*>(lds4);
  for (u32 t = tid; t < kCtlBytes / 4u; t += blockDim.x) ctl[t] = 0u;
  for (u32 t = tid; t < rows_max; t += blockDim.x) ctl[lay.cnt / 4u + t] = 0u;
  __syncthreads();                       // the only workgroup-wide barrier: before the roles split
  if (wave == 0u) {
    producer(entries, count, consumers, lds_base, status);
    return;
  }
  ConsumerState st;
  st.lds_base = lds_base;
  st.ring = lds_base + lay.ring;
  st.consumers = consumers;
  st.me = wave - 1u;
  st.bar_gen = 0u;
  st.stream_kb = 0u;
  st.filled_seen = 0u;
  st.status = status;
  st.spin_limit = spin_limit;
  st.norm_scale = 1.0f;
  st.xr_x = nullptr;
  st.xr_k = 0u;
  st.xr_class = 0u;
  float xr[64], sx[4] = {0.0f, 0.0f, 0.0f, 0.0f}, scale = 1.0f;
#pragma unroll
  for (int i = 0; i < 64; ++i) xr[i] = 0.0f;
  u32 bar = 0u;
  for (u32 i = 0; i < count; ++i) {
    const ChainEntry e = entries[i];
    st.entry_index = i;
    u32* b = (e.flags & CHAIN_BARRIER_BEFORE) ? counters + bar * chain_barrier_stride(gridDim.x) : nullptr;
    const bool same_x = (e.flags & CHAIN_SAME_X) != 0u;
    bool ok = true;
    if (e.fmt == FMT_Q4K) {
      float (&s2)[2] = *reinterpret_cast<float (*)[2]>(&sx[0]);
      ok = consume_entry<FMT_Q4K>(st, e, lay, b, b, same_x, xr, s2, scale);
    } else if (e.fmt == FMT_Q5K) {
      float (&s2)[2] = *reinterpret_cast<float (*)[2]>(&sx[0]);
      ok = consume_entry<FMT_Q5K>(st, e, lay, b, b, same_x, xr, s2, scale);
    } else {
      ok = consume_entry<FMT_Q6K>(st, e, lay, b, b, same_x, xr, sx, scale);
    }
    if (!ok) return;
    if (b) ++bar;
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

}  // namespace stream
