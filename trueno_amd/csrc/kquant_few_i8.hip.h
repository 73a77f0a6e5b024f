// Q4_K product for two to four tokens on the integer matrix cores (gfx950, v_mfma_i32_32x32x32_i8):
//
//   C[m x n] = A[m x k] . dequant(W[n x k])^T,  c[token * n + row]     (trueno-gpu/src/kernels/quantize.rs:568-574;
//   weights decoded as in the GEMV family, quantize.rs:1237-1483), 2 <= m <= 4, k <= 4096.
//
// Why.  The VALU form of the product (one FMA per weight and token, unpacking and scales on top) is what a GEMV is bound
// by, and every further token costs as much again; the f16 matrix-core form pays for its tiles of 16 tokens with a start
// and an end (token conversion, the sum over the parts of K across workgroups) of 8 us.  Here the weights are read once
// for all tokens, the multiply-adds run on the matrix cores, and what is left to the vector unit is one AND per four
// weights and a handful of instructions per (row, sub-block, token).  Measured on MI355X (14336 x 4096, cold weights):
// 10.3 us for two tokens and 12.3 us for four, against 14.8 us for either through the f16 form.  More tokens do not pay:
// every workgroup needs the digits of every token, and with eight that start alone takes 6 us.  Time stamps inside
// the kernel (four tokens, two tiles per workgroup): activations there at 0.8 us, first copies asked for at 1.1 us, digits
// in the registers at 4.9 us, first tile staged at 6.5 us (all 224 workgroups ask for their first 75 KB at once: 16.8 MB),
// 1.4 us to multiply a tile, second tile staged at 8.9 us, end at 11.3 us.
//
// Arithmetic.  For a token t and a run of 256 activations (a super-block's columns) the activations are brought to
// integers X = rint(x * 2^e) with |X| <= 2^30 (e from the run's largest magnitude) and cut into four signed digits of
// eight bits, X = D0 + 256 D1 + 256^2 D2 + 256^3 D3: the bytes of (X + 0x808080) ^ 0x808080.  Per sub-block j (32
// weights) one MFMA forms, exactly, the 32 integers sum_i q_i D_d,i (d = 0..3; 32 operand rows, of which 4 m are in use)
// for 32 rows of W at once; they are joined to S_j = sum_i q_i X_i in f32 (one rounding per join), and the row's share
// of the result is
//   sum_sb 2^-e ( d * sum_j s_j S_j  -  dmin * sum_j m_j SX_j ),   SX_j = sum_i X_i,
// with d, dmin, s_j, m_j the row's own scales (get_scale_min_k4, quantize.rs:1306-1385).  The activations lose what lies
// below 2^-30 of their run's largest element (f32 itself keeps 2^-24 of each element); a sub-block's 32 products are
// summed without rounding, where an f32 evaluation rounds 32 times.
//
// Operand roles (checked against the hardware): lane l supplies A[row l % 32][k = 16 (l / 32) + 0..15] and
// B[k = 16 (l / 32) + 0..15][col l % 32], D[row 8 (v / 4) + 4 (l / 32) + v % 4][col l % 32] arrives in lane l, register
// v.  A = digits, row 4 t + d; B = weights, column = row of W.  A lane so holds ONE row of W - its scales are scalars of
// the lane - and in its sixteen results the four digits of the tokens 2 a + l / 32, a = 0..3.
//
// Data movement.  A workgroup of eight waves takes tiles of 32 rows of W: the rows lie one behind the other in memory
// and are copied as they lie (global_load_lds_dwordx4, non-temporal, every line asked for once) into one of two tile
// buffers in LDS, rows 32 bytes further apart than in memory so that the lanes' 16-byte reads spread over the banks.
// Wave w multiplies the super-blocks 2 w and 2 w + 1 of a tile's rows (its 64 registers of digits cover those 512
// columns for the whole launch): it takes its part of a landed tile into registers, and when every wave has, the
// buffer is given to the tile after next - two tiles are on their way while one is multiplied.  The eight waves' shares
// of a tile meet in LDS (two areas in turn) and are added in wave order while the next tile is multiplied.  The digits
// are made once per workgroup, two tokens at a time, and reach the waves through the upper half of the second tile
// buffer, while the first tile and the lower half of the second are already on their way.  No barrier of the kernel
// waits for copies in flight (wg_barrier).
#pragma once
#include "kquant_common.hip.h"

namespace few_i8 {

typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x16 __attribute__((ext_vector_type(16)));

constexpr u32 kWaves = 8;
constexpr u32 kTileRows = 32;
constexpr u32 kRowPad = 32;                     // LDS bytes between the end of a row and the start of the next
__host__ __device__ constexpr u32 row_stride(u32 nsb) { return nsb * 144u + kRowPad; }
__host__ __device__ constexpr u32 tile_bytes(u32 nsb) { return kTileRows * row_stride(nsb); }
// dynamic LDS: two tile buffers (the upper half of the second holds the digits first), two areas for the waves' partial
// results, the sub-block sums and scales of the tokens
__host__ __device__ constexpr u32 lds_bytes(u32 nsb, u32 ntok) {
  return 2u * tile_bytes(nsb) + 2u * kWaves * kTileRows * ntok * 4u + ntok * nsb * 9u * 4u;
}
// the digits of two tokens on their way to the registers: per half sub-block eight operand rows of 16 bytes
__host__ __device__ constexpr u32 digit_bytes(u32 nsb) { return nsb * 16u * 8u * 16u; }
static_assert(digit_bytes(16) <= tile_bytes(16) / 2u && digit_bytes(1) <= tile_bytes(1) / 2u, "two tokens' digits fit half a tile buffer");
static_assert(lds_bytes(16, 4) <= 160u * 1024u, "LDS of a CU");

__device__ __forceinline__ void lds_r128(u32x4& v, u32 addr) { asm volatile("ds_read_b128 %0, %1" : "=&v"(v) : "v"(addr) : "memory"); }
__device__ __forceinline__ void lds_r32(u32& v, u32 addr) { asm volatile("ds_read_b32 %0, %1" : "=&v"(v) : "v"(addr) : "memory"); }
__device__ __forceinline__ void lds_w128(u32 addr, const u32x4& v) { asm volatile("ds_write_b128 %0, %1" ::"v"(addr), "v"(v) : "memory"); }
__device__ __forceinline__ void lds_w32(u32 addr, u32 v) { asm volatile("ds_write_b32 %0, %1" ::"v"(addr), "v"(v) : "memory"); }
__device__ __forceinline__ void lds_wait() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }
__device__ __forceinline__ void dma16(const uint8_t* src, u32 lds_addr) {
  __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                   (__attribute__((address_space(3))) void*)(uintptr_t)lds_addr, 16, 0, 2 /* nt */);
}
// maximum over the 16 lanes of a DPP row, in every lane of the row
__device__ __forceinline__ u32 row_max_u32(u32 v) {
  v = max(v, static_cast<u32>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0xB1, 0xF, 0xF, true)));
  v = max(v, static_cast<u32>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0x4E, 0xF, 0xF, true)));
  v = max(v, static_cast<u32>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0x141, 0xF, 0xF, true)));
  v = max(v, static_cast<u32>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0x140, 0xF, 0xF, true)));
  return v;
}
// Workgroup barrier over the LDS accesses only (all of them are written in asm here).  __syncthreads() would also wait
// for every copy into LDS that is in flight - the compiler places s_waitcnt vmcnt(0) in front of its barrier - which is
// the one thing the order of the copies is there to avoid.
__device__ __forceinline__ void wg_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }
// at most n of this wave's vector-memory operations outstanding (n <= 14 here)
__device__ __forceinline__ void wait_vm(u32 n) {
  switch (n) {
    case 0: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;
    case 4: asm volatile("s_waitcnt vmcnt(4)" ::: "memory"); break;
    case 5: asm volatile("s_waitcnt vmcnt(5)" ::: "memory"); break;
    case 6: asm volatile("s_waitcnt vmcnt(6)" ::: "memory"); break;
    case 8: asm volatile("s_waitcnt vmcnt(8)" ::: "memory"); break;
    case 9: asm volatile("s_waitcnt vmcnt(9)" ::: "memory"); break;
    case 10: asm volatile("s_waitcnt vmcnt(10)" ::: "memory"); break;
    case 12: asm volatile("s_waitcnt vmcnt(12)" ::: "memory"); break;
    case 13: asm volatile("s_waitcnt vmcnt(13)" ::: "memory"); break;
    case 14: asm volatile("s_waitcnt vmcnt(14)" ::: "memory"); break;
    default: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;
  }
}
// a store that is an instruction of its own on every path (the waits above count it)
__device__ __forceinline__ void store_f32(float* p, float v) {
  asm volatile("global_store_dword %0, %1, off" ::"v"(p), "v"(v) : "memory");
}

// NTOK: tokens the kernel is built for (2 or 4; tokens m .. NTOK - 1 are zeros).  One workgroup: rows
// row0 .. row0 + rows - 1 of W (rows > 0).  lds: byte address of the dynamic LDS.
template <int NTOK>
__device__ __forceinline__ void q4k_rows(const float* __restrict__ a, const uint8_t* __restrict__ w, float* __restrict__ c, u32 m, u32 n,
                                         u32 k, u32 row0, u32 rows, u32 lds) {
  static_assert(NTOK == 2 || NTOK == 4, "two or four tokens");
  constexpr int NA = NTOK / 2;                      // tokens per lane: 2 a + l / 32, a < NA
  constexpr int PHASES = NTOK / 2;                  // the digits are made two tokens at a time
  const u32 tid = threadIdx.x, lane = tid & 63u;
  const u32 wave = static_cast<u32>(__builtin_amdgcn_readfirstlane(static_cast<int>(tid >> 6)));
  const u32 nsb = k >> 8;                           // 1 .. 16
  const u32 row_bytes = nsb * 144u, rs = row_stride(nsb), tb = tile_bytes(nsb);
  const u32 lds_tiles = lds;
  const u32 lds_dig = lds_tiles + tb + 16u * rs;                       // the digits' way to the registers: rows 16 .. 31 of the second buffer
  const u32 red_bytes = kWaves * kTileRows * NTOK * 4u;
  const u32 lds_red = lds + 2u * tb;                                   // [tile parity][wave][row][token] f32
  const u32 lds_sx = lds_red + 2u * red_bytes;                         // [token][sub-block of the row] f32 sums of X
  const u32 lds_fs = lds_sx + NTOK * nsb * 8u * 4u;                    // [token][super-block] f32: 2^-e
  const u32 col = lane & 31u, g = lane >> 5;

  // ---- tile copies ---------------------------------------------------------------------------------------------------
  const u32 tiles = (rows + kTileRows - 1u) / kTileRows;
  const u32 full = row_bytes >> 10, rem16 = (row_bytes & 1023u) >> 4;        // whole KB of a row, 16-byte pieces behind them
  // wave w copies rows 4 w .. 4 w + 3 of a tile: per row `full` instructions of 64 pieces and one of rem16 pieces
  // (144 nsb is never a multiple of 1024 for nsb <= 16: every row has the short copy)
  // (the rows rb .. re - 1 of its four: a wave that issues more copies than the CU can have in flight - about 64 KB - stands
  // still until earlier ones have landed, so the copies of a tile are issued in slices between slices of other work)
  auto issue_rows = [&](u32 tile, u32 rb, u32 re) {
    const u32 buf = lds_tiles + (tile & 1u) * tb;
    for (u32 r = rb; r < re; ++r) {
      const u32 tr = 4u * wave + r;
      u32 row = row0 + tile * kTileRows + tr;
      row = row < n ? row : n - 1u;                  // rows behind the matrix re-read its last row: never stored
      const uint8_t* src = w + static_cast<size_t>(row) * row_bytes + 16u * lane;
      const u32 dst = buf + tr * rs;
      for (u32 j = 0; j < full; ++j) dma16(src + 1024u * j, dst + 1024u * j);
      if (lane < rem16) dma16(src + 1024u * full, dst + 1024u * full);
    }
  };
  auto issue = [&](u32 tile) { issue_rows(tile, 0u, 4u); };
  const u32 per_tile = 4u * (full + 1u);             // copies a wave issues per tile: 4, 8 or 12

  // ---- the digits: 16 lanes convert one (token, super-block) run, 16 values each ------------------------------------
  // thread = (token of the pair tid / 256, half sub-block tid % 256 = 16 sb + q16); phase p converts the tokens 2 p, 2 p + 1.
  // The activations of every phase are asked for first.
  const u32 tt = tid >> 8, half_mine = tid & 255u;
  const bool task = half_mine < nsb * 16u;
  const u32 sb_mine = half_mine >> 4, q16 = half_mine & 15u;
  f32x4 xall[PHASES][4];
#pragma unroll
  for (int ph = 0; ph < PHASES; ++ph) {
    const u32 t = tt + 2u * ph;
    if (task && t < m) {
      const f32x4* src = reinterpret_cast<const f32x4*>(a + static_cast<size_t>(t) * k + half_mine * 16u);
#pragma unroll
      for (int i = 0; i < 4; ++i) xall[ph][i] = src[i];
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) xall[ph][i] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    }
  }
  // The first tile sets out before the digits are made, but behind the activations: loads return in the order they
  // were issued, and the compiler waits for its loads as if the copies were not there.  The second tile's lower half
  // (the waves 0 .. 3) follows at once; its upper half is where the digits pass through.
#pragma unroll
  for (int ph = 0; ph < PHASES; ++ph) asm volatile("" : "+v"(xall[ph][0]), "+v"(xall[ph][1]), "+v"(xall[ph][2]), "+v"(xall[ph][3])::"memory");
  issue_rows(0u, 0u, 2u);
  i32x4 dig[16];
#pragma unroll
  for (int js = 0; js < 16; ++js) dig[js] = i32x4{0, 0, 0, 0};
#pragma unroll
  for (int ph = 0; ph < PHASES; ++ph) {
    if (task) {
      const u32 t = tt + 2u * ph;
      const f32x4* xv = xall[ph];
      u32 amax = 0u;
#pragma unroll
      for (int i = 0; i < 4; ++i)
        amax = max(max(amax, __float_as_uint(xv[i].x) & 0x7FFFFFFFu),
                   max(max(__float_as_uint(xv[i].y) & 0x7FFFFFFFu, __float_as_uint(xv[i].z) & 0x7FFFFFFFu), __float_as_uint(xv[i].w) & 0x7FFFFFFFu));
      amax = row_max_u32(amax);
      u32 eb = amax >> 23;                           // biased exponent of the run's largest magnitude: |x| < 2^(eb - 126)
      const bool finite = eb != 255u;
      eb = eb < 30u ? 30u : eb;                      // keeps both powers of two normal numbers
      const float up = __uint_as_float((283u - eb) << 23);       // 2^(156 - eb): |x| * up < 2^30
      // X + 0x808080 has the bytes D + 128 (D3 as it is): the xor makes signed bytes of them.  Then the 4 x 4 bytes of four
      // values are transposed: plane[d] word v = digit d of the values 4 v .. 4 v + 3.
      u32x4 plane[4];
      int dsum[4] = {0, 0, 0, 0};
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const float xs[4] = {xv[v].x, xv[v].y, xv[v].z, xv[v].w};
        u32 z[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) z[i] = (static_cast<u32>(static_cast<int>(__builtin_rintf(xs[i] * up))) + 0x00808080u) ^ 0x00808080u;
        const u32 t0 = __builtin_amdgcn_perm(z[1], z[0], 0x05010400u), t1 = __builtin_amdgcn_perm(z[1], z[0], 0x07030602u);
        const u32 u0 = __builtin_amdgcn_perm(z[3], z[2], 0x05010400u), u1 = __builtin_amdgcn_perm(z[3], z[2], 0x07030602u);
        plane[0][v] = __builtin_amdgcn_perm(u0, t0, 0x05040100u);
        plane[1][v] = __builtin_amdgcn_perm(u0, t0, 0x07060302u);
        plane[2][v] = __builtin_amdgcn_perm(u1, t1, 0x05040100u);
        plane[3][v] = __builtin_amdgcn_perm(u1, t1, 0x07060302u);
#pragma unroll
        for (int d = 0; d < 4; ++d) dsum[d] = __builtin_amdgcn_sdot4(static_cast<int>(plane[d][v]), 0x01010101, dsum[d], false);
      }
      // Consumer: half sub-block `half_mine` of the row, operand row 4 (token of the pair) + d of the eight of this phase.
      // The eight rows of a half sub-block lie 16 bytes apart in an order rotated by the half sub-block's number, so that
      // the sixteen lanes that write one row of sixteen neighbouring half sub-blocks do not all hit the same banks.
      const u32 dst = lds_dig + half_mine * 128u;
#pragma unroll
      for (u32 d = 0; d < 4u; ++d) lds_w128(dst + (((4u * tt + d) ^ half_mine) & 7u) * 16u, plane[d]);
      // SX of the sub-block: the digits' sums over its 32 values (with the neighbour's half), joined in f32
#pragma unroll
      for (int d = 0; d < 4; ++d) dsum[d] += __builtin_amdgcn_update_dpp(0, dsum[d], 0xB1, 0xF, 0xF, true);
      const float sx = fmaf(static_cast<float>(dsum[3]), 16777216.0f, fmaf(static_cast<float>(dsum[2]), 65536.0f,
                            fmaf(static_cast<float>(dsum[1]), 256.0f, static_cast<float>(dsum[0]))));
      if ((q16 & 1u) == 0u) lds_w32(lds_sx + (t * nsb * 8u + sb_mine * 8u + (q16 >> 1)) * 4u, __float_as_uint(sx));
      if (q16 == 0u) lds_w32(lds_fs + (t * nsb + sb_mine) * 4u, finite ? (eb - 29u) << 23 : 0x7FC00000u);      // 2^(eb - 156) = 1 / up
    }
    // the next slice of copies: the rest of the first tile, then the lower half of the second (rows 0 .. 15: the waves
    // 0 .. 3), whose upper half is where the digits pass through
    if (ph == 0) issue_rows(0u, 2u, 4u);
    if (ph == PHASES - 1 && wave < 4u && tiles > 1u) issue_rows(1u, 0u, 2u);
    wg_barrier();
    // this wave's digits of this phase's tokens: sub-blocks 0 .. 15 of its two super-blocks, operand row col (= 4 t + d)
    // and half g of the sub-block; operand rows of tokens the kernel is not built for stay zero
    if ((col >> 3) == static_cast<u32>(ph)) {
      u32x4 raw[16];
#pragma unroll
      for (u32 js = 0; js < 16u; ++js) {
        const u32 half = (wave * 16u + js) * 2u + g;
        if (wave * 16u + js < nsb * 8u) lds_r128(raw[js], lds_dig + half * 128u + (((col & 7u) ^ half) & 7u) * 16u);
        else raw[js] = u32x4{0u, 0u, 0u, 0u};
      }
      lds_wait();
#pragma unroll
      for (int js = 0; js < 16; ++js) {
        asm volatile("" : "+v"(raw[js]));
        dig[js] = __builtin_bit_cast(i32x4, raw[js]);
      }
    }
    wg_barrier();                                    // the digits are read: the next phase's, or the tile's rows, may come
  }
  if (tiles > 1u) {
    if (wave < 4u) issue_rows(1u, 2u, 4u);
    else issue(1u);
  }

  // ---- tiles --------------------------------------------------------------------------------------------------------
  // A tile's results leave while the next tile is multiplied: every wave adds up its share of them (4 NTOK of the
  // 32 NTOK) and issues ONE store per tile, by every lane (lanes without a result of their own repeat a neighbour's),
  // so that the number of this wave's memory operations behind a tile's copies is known: the next tile's copies and the
  // stores issued since.
  const bool active0 = 2u * wave < nsb, active1 = 2u * wave + 1u < nsb;
  auto reduce_store = [&](u32 tile) {
    const u32 o = wave * (4u * NTOK) + (lane & (4u * NTOK - 1u));
    const u32 valid = min(kTileRows, rows - tile * kTileRows);      // rows of this tile that exist (>= 1)
    u32 r = o / NTOK, t = o & (NTOK - 1u);
    r = r < valid ? r : valid - 1u;
    t = t < m ? t : m - 1u;
    const u32 from = lds_red + (tile & 1u) * red_bytes + (r * NTOK + t) * 4u;
    u32 part[kWaves];
#pragma unroll
    for (u32 wv = 0; wv < kWaves; ++wv) lds_r32(part[wv], from + wv * kTileRows * NTOK * 4u);
    lds_wait();
    float sum = 0.0f;
#pragma unroll
    for (u32 wv = 0; wv < kWaves; ++wv) {
      asm volatile("" : "+v"(part[wv]));
      if (2u * wv < nsb) sum += __uint_as_float(part[wv]);
    }
    store_f32(c + static_cast<size_t>(t) * n + (row0 + tile * kTileRows + r), sum);
  };
  for (u32 tile = 0; tile < tiles; ++tile) {
    // tile `tile` has landed when no more of this wave's operations are outstanding than were issued behind its copies:
    // the next tile's copies, and the store of the tile tile - 2 (issued in the round before, ahead of those copies)
    wait_vm(tile + 1u < tiles ? per_tile + (tile >= 2u ? 1u : 0u) : 0u);
    wg_barrier();
    // this wave's part of the tile goes to registers, so that the buffer can take the tile after next while this one is
    // multiplied: two tiles on their way at any time
    const u32 rowp = lds_tiles + (tile & 1u) * tb + col * rs + 2u * wave * 144u;
    u32x4 hdr2[2], pc2[2][4];
#pragma unroll
    for (u32 sbi = 0; sbi < 2u; ++sbi) {
      if (!(sbi == 0u ? active0 : active1)) continue;
      lds_r128(hdr2[sbi], rowp + sbi * 144u);
#pragma unroll
      for (u32 ch = 0; ch < 4u; ++ch) lds_r128(pc2[sbi][ch], rowp + sbi * 144u + 16u + 32u * ch + 16u * g);
    }
    lds_wait();
#pragma unroll
    for (u32 sbi = 0; sbi < 2u; ++sbi)
      if (sbi == 0u ? active0 : active1)
        asm volatile("" : "+v"(hdr2[sbi]), "+v"(pc2[sbi][0]), "+v"(pc2[sbi][1]), "+v"(pc2[sbi][2]), "+v"(pc2[sbi][3]));
    wg_barrier();                                    // every wave has its part (and wrote its share of the tile before): the buffer is free
    const bool more = tile + 2u < tiles;             // the tile after next: its copies are issued a row at a time between the MFMAs below
    if (tile > 0u) reduce_store(tile - 1u);
    if (more && !active0) issue(tile + 2u);          // (a wave without a super-block of its own has no MFMAs to put them between)
    float y[NA];
#pragma unroll
    for (int aa = 0; aa < NA; ++aa) y[aa] = 0.0f;
#pragma unroll
    for (u32 sbi = 0; sbi < 2u; ++sbi) {
      if (!(sbi == 0u ? active0 : active1)) continue;
      const u32 sb = 2u * wave + sbi;
      const u32x4 hdr = hdr2[sbi], pc[4] = {pc2[sbi][0], pc2[sbi][1], pc2[sbi][2], pc2[sbi][3]};
      // the sums and scales of this lane's tokens (the same for all rows: broadcast reads)
      u32x4 sxa[NA][2];
      u32 fsa[NA];
#pragma unroll
      for (int aa = 0; aa < NA; ++aa) {
        const u32 t = 2u * aa + g;
        lds_r128(sxa[aa][0], lds_sx + (t * nsb * 8u + sb * 8u) * 4u);
        lds_r128(sxa[aa][1], lds_sx + (t * nsb * 8u + sb * 8u + 4u) * 4u);
        lds_r32(fsa[aa], lds_fs + (t * nsb + sb) * 4u);
      }
      lds_wait();
#pragma unroll
      for (int aa = 0; aa < NA; ++aa) asm volatile("" : "+v"(sxa[aa][0]), "+v"(sxa[aa][1]), "+v"(fsa[aa]));
      // the row's scales: get_scale_min_k4 (quantize.rs:1306-1385), sub-blocks 0..3 and 4..7 as bytes of two words each
      const float d = half_bits_to_f32(hdr.x), dmin = half_bits_to_f32(hdr.x >> 16);
      const u32 s_lo = hdr.y & 0x3F3F3F3Fu, m_lo = hdr.z & 0x3F3F3F3Fu;
      const u32 s_hi = (hdr.w & 0x0F0F0F0Fu) | ((hdr.y >> 2) & 0x30303030u);
      const u32 m_hi = ((hdr.w >> 4) & 0x0F0F0F0Fu) | ((hdr.z >> 2) & 0x30303030u);
      float P[NA], Q[NA];
#pragma unroll
      for (int aa = 0; aa < NA; ++aa) P[aa] = Q[aa] = 0.0f;
#pragma unroll
      for (u32 ch = 0; ch < 4u; ++ch) {
        const u32 sw = ch < 2u ? s_lo : s_hi, mw = ch < 2u ? m_lo : m_hi;      // sub-blocks 2 ch, 2 ch + 1: bytes 2 (ch % 2), + 1
        const float s0 = static_cast<float>((sw >> (16u * (ch & 1u))) & 0xFFu), s1 = static_cast<float>((sw >> (16u * (ch & 1u) + 8u)) & 0xFFu);
        const float m0 = static_cast<float>((mw >> (16u * (ch & 1u))) & 0xFFu), m1 = static_cast<float>((mw >> (16u * (ch & 1u) + 8u)) & 0xFFu);
        const i32x4 blo = {static_cast<int>(pc[ch].x & 0x0F0F0F0Fu), static_cast<int>(pc[ch].y & 0x0F0F0F0Fu),
                           static_cast<int>(pc[ch].z & 0x0F0F0F0Fu), static_cast<int>(pc[ch].w & 0x0F0F0F0Fu)};
        const i32x4 bhi = {static_cast<int>((pc[ch].x >> 4) & 0x0F0F0F0Fu), static_cast<int>((pc[ch].y >> 4) & 0x0F0F0F0Fu),
                           static_cast<int>((pc[ch].z >> 4) & 0x0F0F0F0Fu), static_cast<int>((pc[ch].w >> 4) & 0x0F0F0F0Fu)};
        const i32x16 zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        if (more && sbi == 0u) issue_rows(tile + 2u, ch, ch + 1u);
        const i32x16 dlo = __builtin_amdgcn_mfma_i32_32x32x32_i8(dig[8 * sbi + 2 * ch], blo, zero, 0, 0, 0);
        const i32x16 dhi = __builtin_amdgcn_mfma_i32_32x32x32_i8(dig[8 * sbi + 2 * ch + 1], bhi, zero, 0, 0, 0);
#pragma unroll
        for (int aa = 0; aa < NA; ++aa) {
          // S = D0 + 256 D1 + 256^2 D2 + 256^3 D3: every term exact in f32, the joins round
          const float lo = fmaf(static_cast<float>(dlo[4 * aa + 3]), 16777216.0f, fmaf(static_cast<float>(dlo[4 * aa + 2]), 65536.0f,
                                fmaf(static_cast<float>(dlo[4 * aa + 1]), 256.0f, static_cast<float>(dlo[4 * aa]))));
          const float hi = fmaf(static_cast<float>(dhi[4 * aa + 3]), 16777216.0f, fmaf(static_cast<float>(dhi[4 * aa + 2]), 65536.0f,
                                fmaf(static_cast<float>(dhi[4 * aa + 1]), 256.0f, static_cast<float>(dhi[4 * aa]))));
          P[aa] = fmaf(s1, hi, fmaf(s0, lo, P[aa]));
          const u32x4 sxw = sxa[aa][ch >> 1];
          const float sx0 = __uint_as_float((ch & 1u) ? sxw.z : sxw.x), sx1 = __uint_as_float((ch & 1u) ? sxw.w : sxw.y);
          Q[aa] = fmaf(m1, sx1, fmaf(m0, sx0, Q[aa]));
        }
      }
#pragma unroll
      for (int aa = 0; aa < NA; ++aa) {
        const float f = __uint_as_float(fsa[aa]);
        y[aa] += fmaf(-(dmin * f), Q[aa], (d * f) * P[aa]);
      }
    }
    // the waves' shares of the tile meet in LDS: red[tile parity][wave][row][token]; they are added up behind the next
    // tile's barriers (or behind the loop), which every wave reaches after these writes
#pragma unroll
    for (int aa = 0; aa < NA; ++aa)
      lds_w32(lds_red + (tile & 1u) * red_bytes + ((wave * kTileRows + col) * NTOK + 2u * aa + g) * 4u, __float_as_uint(y[aa]));
  }
  wg_barrier();
  reduce_store(tiles - 1u);
}

}  // namespace few_i8
