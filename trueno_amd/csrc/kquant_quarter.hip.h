// Quarter-block decoders: the unit of work of the fast kernels.
//
// A lane owns one quarter (64 values) of one 256-value super-block: 4 lanes per super-block,
// 16 super-blocks (4096 values) per wave64.  For each format this file says
//   * which bytes the lane streams from HBM (128-bit loads wherever the layout allows),
//   * how the scale/min fields and the 4/5/6-bit quants are unpacked in registers,
//   * which 64 activations the lane needs (value_index) and how the activation vector is
//     swizzled in LDS so that the wave's 128-bit LDS reads are bank-conflict free,
//   * dot(): sum over the quarter of w*x in the factorised form
//         sum_j ( (d*s_j) * sum_{i in j} q_i x_i  -  (dmin*m_j) * sum_{i in j} x_i ),
//   * dequant(): the 64 f32 weights, with the reference's instruction sequence.
// Decode arithmetic: trueno-gpu/src/kernels/quantize.rs:1237-1483 (Q4_K), :1589-1693 (Q5_K),
// :1806-1934 (Q6_K).
#pragma once
#include "kquant_common.hip.h"

template <int FMT> struct Quarter;

// LDS reads written in asm: a row batch streamed into LDS by DMA is still arriving while the previous one is read, and
// for LDS accesses the compiler can see it waits until every such copy has landed.  The caller waits (lgkmcnt) and then
// passes the registers through landed().
template <int OFF> __device__ __forceinline__ void ldsq_read128(u32x4& v, u32 addr) {
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=&v"(v) : "v"(addr), "n"(OFF) : "memory");
}
template <int OFF> __device__ __forceinline__ void ldsq_read64(u32x2& v, u32 addr) {
  asm volatile("ds_read_b64 %0, %1 offset:%2" : "=&v"(v) : "v"(addr), "n"(OFF) : "memory");
}
template <int OFF> __device__ __forceinline__ void ldsq_read32(u32& v, u32 addr) {
  asm volatile("ds_read_b32 %0, %1 offset:%2" : "=&v"(v) : "v"(addr), "n"(OFF) : "memory");
}
template <int OFF> __device__ __forceinline__ void ldsq_read16(u32& v, u32 addr) {
  asm volatile("ds_read_u16 %0, %1 offset:%2" : "=&v"(v) : "v"(addr), "n"(OFF) : "memory");
}

// ------------------------------------------------------------------------------------------
// Q4_K: quarter c holds qs[32c .. 32c+31]; low nibbles are values 64c+0..31 (sub-block 2c),
// high nibbles are values 64c+32..63 (sub-block 2c+1).
// ------------------------------------------------------------------------------------------
template <> struct Quarter<FMT_Q4K> {
  static constexpr u32 SB = 144;
  static constexpr int NSUM = 2;  // activation sums per quarter: one per sub-block
  struct Regs { u32x4 hdr, q0, q1; };

  static __device__ __forceinline__ u32 swz(u32 unit) { return unit ^ ((unit >> 4) & 15u); }
  static __device__ __forceinline__ u32 value_index(u32 c, u32 j) { return 64u * c + j; }
  static __device__ __forceinline__ u32 sum_index(u32 j) { return j >> 5; }

  // The block lies `off` bytes behind `base`.  Callers hand in a base that is the same for the whole wave (a row of
  // the matrix) and keep what differs from lane to lane in the 32-bit offset: the address of a load is then a scalar
  // register pair plus one vector register, not a 64-bit sum per lane and piece.
  static __device__ __forceinline__ void load(Regs& r, const uint8_t* base, u32 off, u32 c) {
    r.hdr = load128(base + off);
    r.q0 = load128(base + (off + 32u * c) + 16);
    r.q1 = load128(base + (off + 32u * c) + 32);
  }

  // the same three pieces from a copy of the block in LDS (at byte address `blk`)
  static __device__ __forceinline__ void load_lds(Regs& r, u32 blk, u32 c) {
    ldsq_read128<0>(r.hdr, blk);
    ldsq_read128<16>(r.q0, blk + 32u * c);
    ldsq_read128<32>(r.q1, blk + 32u * c);
  }
  static __device__ __forceinline__ void landed(Regs& r) { asm volatile("" : "+v"(r.hdr), "+v"(r.q0), "+v"(r.q1)); }

  // (d*s, dmin*m) for sub-blocks 2c and 2c+1; get_scale_min_k4 packing (quantize.rs:1306-1385).
  static __device__ __forceinline__ void scales(const Regs& r, u32 c, float& ds0, float& ds1, float& dm0, float& dm1) {
    const float d = half_bits_to_f32(r.hdr.x);
    const float dmin = half_bits_to_f32(r.hdr.x >> 16);
    const u32 sh = 16u * (c & 1u);
    const u32 h1 = r.hdr.y >> sh, h2 = r.hdr.z >> sh, h3 = r.hdr.w >> sh;
    // sub-blocks 0..3: s = sc[j] & 63, m = sc[j+4] & 63
    const u32 sp_lo = h1 & 0x3F3Fu, mp_lo = h2 & 0x3F3Fu;
    // sub-blocks 4..7: s = (sc[j+4] & 15) | (sc[j-4] >> 6) << 4,  m = (sc[j+4] >> 4) | (sc[j] >> 6) << 4
    const u32 sp_hi = (h3 & 0x0F0Fu) | ((h1 >> 2) & 0x3030u);
    const u32 mp_hi = ((h3 >> 4) & 0x0F0Fu) | ((h2 >> 2) & 0x3030u);
    const u32 sp = (c & 2u) ? sp_hi : sp_lo;
    const u32 mp = (c & 2u) ? mp_hi : mp_lo;
    ds0 = __fmul_rn(d, ubyte0(sp));
    ds1 = __fmul_rn(d, ubyte1(sp));
    dm0 = __fmul_rn(dmin, ubyte0(mp));
    dm1 = __fmul_rn(dmin, ubyte1(mp));
  }

  // The quants enter the FMAs without an integer-to-float conversion: a 4-bit quant q left in the low bits of a
  // 16-bit lane IS the f16 subnormal q * 2^-24 (in bits 4..7: q * 2^-20), and v_fma_mix_f32 takes an f16 operand.
  // One AND therefore prepares two values.  The products and the running sums are the old ones times 2^-24, a
  // power of two, so every rounding is the same and the factor goes into the scale at the end.
  static __device__ __forceinline__ float dot(const Regs& r, u32 c, const float (&xr)[64], const float (&sx)[NSUM]) {
    float ds0, ds1, dm0, dm1;
    scales(r, c, ds0, ds1, dm0, dm1);
    // Each sub-block's 32 products go into four chains of eight, joined pairwise: no chain is longer than the
    // reference's (eight FMAs per lane and super-block, quantize.rs:1412, 1482), so no partial sum grows larger
    // before it is rounded.  lo accumulates 2^-24 * q x, hi 2^-20 * q x.
    float lo[4] = {0.0f, 0.0f, 0.0f, 0.0f}, hi[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int t = 0; t < 8; ++t) {
      const u32 v = t < 4 ? r.q0[t] : r.q1[t - 4];
      const u32 w = v >> 8;
      const h16x2 l02 = as_h16x2(v & 0x000F000Fu), h02 = as_h16x2(v & 0x00F000F0u);   // bytes 0 and 2
      const h16x2 l13 = as_h16x2(w & 0x000F000Fu), h13 = as_h16x2(w & 0x00F000F0u);   // bytes 1 and 3
      float& l = lo[t & 3];
      float& h = hi[t & 3];
      l = fmaf(static_cast<float>(l02.x), xr[4 * t + 0], l);
      l = fmaf(static_cast<float>(l13.x), xr[4 * t + 1], l);
      l = fmaf(static_cast<float>(l02.y), xr[4 * t + 2], l);
      l = fmaf(static_cast<float>(l13.y), xr[4 * t + 3], l);
      h = fmaf(static_cast<float>(h02.x), xr[32 + 4 * t + 0], h);
      h = fmaf(static_cast<float>(h13.x), xr[32 + 4 * t + 1], h);
      h = fmaf(static_cast<float>(h02.y), xr[32 + 4 * t + 2], h);
      h = fmaf(static_cast<float>(h13.y), xr[32 + 4 * t + 3], h);
    }
    float acc = (ds0 * 16777216.0f) * ((lo[0] + lo[1]) + (lo[2] + lo[3]));
    acc = fmaf(ds1 * 1048576.0f, (hi[0] + hi[1]) + (hi[2] + hi[3]), acc);
    acc = fmaf(-dm0, sx[0], acc);
    acc = fmaf(-dm1, sx[1], acc);
    return acc;
  }

  static __device__ __forceinline__ void dequant(const Regs& r, u32 c, float (&w)[64]) {
    float ds0, ds1, dm0, dm1;
    scales(r, c, ds0, ds1, dm0, dm1);
#pragma unroll
    for (int t = 0; t < 8; ++t) {
      const u32 v = t < 4 ? r.q0[t] : r.q1[t - 4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const u32 byte = (v >> (8 * i)) & 0xFFu;
        w[4 * t + i] = __fsub_rn(__fmul_rn(ds0, static_cast<float>(byte & 15u)), dm0);
        w[32 + 4 * t + i] = __fsub_rn(__fmul_rn(ds1, static_cast<float>(byte >> 4)), dm1);
      }
    }
  }
};

// ------------------------------------------------------------------------------------------
// Q5_K (the reference's own layout): nibbles as Q4_K; fifth bit of value i is bit i%8 of
// qh[i/8], so quarter c owns qh[8c .. 8c+7]; scales are contiguous 12-bit fields, so quarter c
// owns the 24 bits starting at byte 3c of sc[].
// ------------------------------------------------------------------------------------------
template <> struct Quarter<FMT_Q5K> {
  static constexpr u32 SB = 176;
  static constexpr int NSUM = 2;
  struct Regs { u32 dd, f24; u32x4 q0, q1; u32x2 qh; };

  static __device__ __forceinline__ u32 swz(u32 unit) { return unit ^ ((unit >> 4) & 15u); }
  static __device__ __forceinline__ u32 value_index(u32 c, u32 j) { return 64u * c + j; }
  static __device__ __forceinline__ u32 sum_index(u32 j) { return j >> 5; }

  static __device__ __forceinline__ void load(Regs& r, const uint8_t* base, u32 off, u32 c) {
    r.dd = load32(base + off);
    r.f24 = load32_a1(base + (off + 3u * c) + 4);  // c == 3 also reads qs[0]; masked off below
    r.q0 = load128(base + (off + 32u * c) + 16);
    r.q1 = load128(base + (off + 32u * c) + 32);
    r.qh = load64(base + (off + 8u * c) + 144);
  }

  static __device__ __forceinline__ void load_lds(Regs& r, u32 blk, u32 c) {
    ldsq_read32<0>(r.dd, blk);
    ldsq_read32<4>(r.f24, blk + 3u * c);         // at any byte alignment, like the load from memory
    ldsq_read128<16>(r.q0, blk + 32u * c);
    ldsq_read128<32>(r.q1, blk + 32u * c);
    ldsq_read64<144>(r.qh, blk + 8u * c);
  }
  static __device__ __forceinline__ void landed(Regs& r) { asm volatile("" : "+v"(r.dd), "+v"(r.f24), "+v"(r.q0), "+v"(r.q1), "+v"(r.qh)); }

  static __device__ __forceinline__ void scales(const Regs& r, float& ds0, float& ds1, float& dm0, float& dm1) {
    const float d = half_bits_to_f32(r.dd);
    const float dmin = half_bits_to_f32(r.dd >> 16);
    const u32 f = r.f24;                                       // quantize.rs:1607-1635
    ds0 = __fmul_rn(d, static_cast<float>(f & 63u));
    dm0 = __fmul_rn(dmin, static_cast<float>((f >> 6) & 63u));
    ds1 = __fmul_rn(d, static_cast<float>((f >> 12) & 63u));
    dm1 = __fmul_rn(dmin, static_cast<float>((f >> 18) & 63u));
  }

  // four 5-bit quants as the four bytes of a word: nibbles | (bit << 4).  `bits4` holds the four
  // fifth-bits in bits 4..7; the 24-bit multiply copies bit 4+i to bit 4+8i (no carries).
  static __device__ __forceinline__ u32 join5(u32 nibbles, u32 bits4) {
    return (__umul24(bits4, 0x204081u) & 0x10101010u) | nibbles;
  }

  // As for Q4_K the quants enter the FMAs as f16 subnormals: a 5-bit quant in the low bits of a 16-bit lane is
  // q * 2^-24, and v_fma_mix_f32 takes it as it is; the factor leaves through the scale, every rounding unchanged.
  static __device__ __forceinline__ float dot(const Regs& r, u32 c, const float (&xr)[64], const float (&sx)[NSUM]) {
    float ds0, ds1, dm0, dm1;
    scales(r, ds0, ds1, dm0, dm1);
    float lo[4] = {0.0f, 0.0f, 0.0f, 0.0f}, hi[4] = {0.0f, 0.0f, 0.0f, 0.0f};   // four chains of eight per sub-block, as for Q4_K
#pragma unroll
    for (int t = 0; t < 8; ++t) {
      const u32 v = t < 4 ? r.q0[t] : r.q1[t - 4];
      const u32 bl = t == 0 ? (r.qh.x << 4) & 0xF0u : (r.qh.x >> (4 * t - 4)) & 0xF0u;
      const u32 bh = t == 0 ? (r.qh.y << 4) & 0xF0u : (r.qh.y >> (4 * t - 4)) & 0xF0u;
      const u32 l = opaque(join5(v & 0x0F0F0F0Fu, bl));
      const u32 h = opaque(join5((v >> 4) & 0x0F0F0F0Fu, bh));
      const h16x2 l02 = as_h16x2(l & 0x001F001Fu), l13 = as_h16x2((l >> 8) & 0x001F001Fu);   // bytes 0,2 and 1,3
      const h16x2 h02 = as_h16x2(h & 0x001F001Fu), h13 = as_h16x2((h >> 8) & 0x001F001Fu);
      float& lc = lo[t & 3];
      float& hc = hi[t & 3];
      lc = fmaf(static_cast<float>(l02.x), xr[4 * t + 0], lc);
      lc = fmaf(static_cast<float>(l13.x), xr[4 * t + 1], lc);
      lc = fmaf(static_cast<float>(l02.y), xr[4 * t + 2], lc);
      lc = fmaf(static_cast<float>(l13.y), xr[4 * t + 3], lc);
      hc = fmaf(static_cast<float>(h02.x), xr[32 + 4 * t + 0], hc);
      hc = fmaf(static_cast<float>(h13.x), xr[32 + 4 * t + 1], hc);
      hc = fmaf(static_cast<float>(h02.y), xr[32 + 4 * t + 2], hc);
      hc = fmaf(static_cast<float>(h13.y), xr[32 + 4 * t + 3], hc);
    }
    float acc = (ds0 * 16777216.0f) * ((lo[0] + lo[1]) + (lo[2] + lo[3]));
    acc = fmaf(ds1 * 16777216.0f, (hi[0] + hi[1]) + (hi[2] + hi[3]), acc);
    acc = fmaf(-dm0, sx[0], acc);
    acc = fmaf(-dm1, sx[1], acc);
    return acc;
  }

  static __device__ __forceinline__ void dequant(const Regs& r, u32 c, float (&w)[64]) {
    float ds0, ds1, dm0, dm1;
    scales(r, ds0, ds1, dm0, dm1);
#pragma unroll
    for (int t = 0; t < 8; ++t) {
      const u32 v = t < 4 ? r.q0[t] : r.q1[t - 4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const u32 byte = (v >> (8 * i)) & 0xFFu;
        const u32 ql = (byte & 15u) + 16u * ((r.qh.x >> (4 * t + i)) & 1u);
        const u32 qhv = (byte >> 4) + 16u * ((r.qh.y >> (4 * t + i)) & 1u);
        w[4 * t + i] = __fsub_rn(__fmul_rn(ds0, static_cast<float>(ql)), dm0);
        w[32 + 4 * t + i] = __fsub_rn(__fmul_rn(ds1, static_cast<float>(qhv)), dm1);
      }
    }
  }
};

// ------------------------------------------------------------------------------------------
// Q6_K: quarter c = (h = c/2, is = c%2) owns l = 16*is .. 16*is+15 of half h:
//   A = ql[64h + l]      low nibble -> group 0 (value 128h + l),      high -> group 2 (+64)
//   B = ql[64h + 32 + l] low nibble -> group 1 (value 128h + 32 + l), high -> group 3 (+96)
//   C = qh[32h + l]      bits 2g..2g+1 -> group g
//   scale of group g = sc[8h + is + 2g] (int8).  Blocks are only 2-byte aligned.
// x register j = 16g + t  <->  value 128h + 32g + 16is + t.
// ------------------------------------------------------------------------------------------
template <> struct Quarter<FMT_Q6K> {
  static constexpr u32 SB = 210;
  static constexpr int NSUM = 4;  // one per group of 16
  struct Regs { u32x4 a, b, c; u32x2 sc; u32 d; };

  static __device__ __forceinline__ u32 swz(u32 unit) {
    return unit ^ ((unit >> 6) & 3u) ^ (((unit >> 5) & 1u) << 3);
  }
  static __device__ __forceinline__ u32 value_index(u32 c, u32 j) {
    return 128u * (c >> 1) + 32u * (j >> 4) + 16u * (c & 1u) + (j & 15u);
  }
  static __device__ __forceinline__ u32 sum_index(u32 j) { return j >> 4; }

  static __device__ __forceinline__ void load(Regs& r, const uint8_t* base, u32 off, u32 c) {
    const u32 h = c >> 1, is = c & 1u;
    r.a = load128_a2(base + (off + 64u * h + 16u * is));
    r.b = load128_a2(base + (off + 64u * h + 16u * is) + 32);
    r.c = load128_a2(base + (off + 32u * h + 16u * is) + 128);
    r.sc = load64_a2(base + (off + 8u * h) + 192);
    r.d = load16_a2(base + off + 208);
  }

  // From the copy in LDS, where the block starts on a 16-byte boundary and its last 16 bytes (194..209) lie at 208: d
  // is the half word at 222.
  static __device__ __forceinline__ void load_lds(Regs& r, u32 blk, u32 c) {
    const u32 h = c >> 1, is = c & 1u;
    ldsq_read128<0>(r.a, blk + 64u * h + 16u * is);
    ldsq_read128<32>(r.b, blk + 64u * h + 16u * is);
    ldsq_read128<128>(r.c, blk + 32u * h + 16u * is);
    ldsq_read64<192>(r.sc, blk + 8u * h);
    ldsq_read16<222>(r.d, blk);
  }
  static __device__ __forceinline__ void landed(Regs& r) { asm volatile("" : "+v"(r.a), "+v"(r.b), "+v"(r.c), "+v"(r.sc), "+v"(r.d)); }

  static __device__ __forceinline__ void scales(const Regs& r, u32 c, float (&dsc)[4]) {
    const float d = half_bits_to_f32(r.d);
    const u32 sh = 8u * (c & 1u);
    const int s0 = static_cast<int8_t>((r.sc.x >> sh) & 0xFFu);
    const int s1 = static_cast<int8_t>((r.sc.x >> (sh + 16)) & 0xFFu);
    const int s2 = static_cast<int8_t>((r.sc.y >> sh) & 0xFFu);
    const int s3 = static_cast<int8_t>((r.sc.y >> (sh + 16)) & 0xFFu);
    dsc[0] = __fmul_rn(d, static_cast<float>(s0));
    dsc[1] = __fmul_rn(d, static_cast<float>(s1));
    dsc[2] = __fmul_rn(d, static_cast<float>(s2));
    dsc[3] = __fmul_rn(d, static_cast<float>(s3));
  }

  // the four 6-bit quants (0..63, before the -32) of group g for bytes 4t..4t+3, one per byte
  static __device__ __forceinline__ void quants(const Regs& r, int t, u32 (&q)[4]) {
    const u32 a = r.a[t], b = r.b[t], cc = r.c[t];
    q[0] = opaque((a & 0x0F0F0F0Fu) | ((cc << 4) & 0x30303030u));
    q[1] = opaque((b & 0x0F0F0F0Fu) | ((cc << 2) & 0x30303030u));
    q[2] = opaque(((a >> 4) & 0x0F0F0F0Fu) | (cc & 0x30303030u));
    q[3] = opaque(((b >> 4) & 0x0F0F0F0Fu) | ((cc >> 2) & 0x30303030u));
  }

  // Four signed bytes 4*(q - 32) of group g for bytes 4t..4t+3.  q - 32 is the 6-bit two's complement number
  // q ^ 32; placed in bits 2..7 of a byte its sign-extension is 4*(q - 32), and flipping bit 5 of q is flipping
  // the high bit of its 2-bit field in qh, which is done once per qh word (`cx` = qh ^ 0xAAAAAAAA).
  static __device__ __forceinline__ void quants_s4(const Regs& r, int t, u32 cx, u32 (&q)[4]) {
    const u32 a = r.a[t], b = r.b[t];
    q[0] = ((a << 2) & 0x3C3C3C3Cu) | ((cx << 6) & 0xC0C0C0C0u);
    q[1] = ((b << 2) & 0x3C3C3C3Cu) | ((cx << 4) & 0xC0C0C0C0u);
    q[2] = ((a >> 2) & 0x3C3C3C3Cu) | ((cx << 2) & 0xC0C0C0C0u);
    q[3] = ((b >> 2) & 0x3C3C3C3Cu) | (cx & 0xC0C0C0C0u);
  }
  static __device__ __forceinline__ float sbyte(u32 v, int i) {
    return static_cast<float>(static_cast<int>(static_cast<int8_t>((v >> (8 * i)) & 0xFFu)));
  }

  // (q - 32) is formed before the multiply: summing q*x and correcting by -32*sum(x) afterwards doubles the
  // rounding error (the two sums are about twice the size of their difference).  It enters as the signed byte
  // 4*(q - 32), converted with its sign in one instruction; the factor 4 is a power of two and leaves through
  // the scale, so every rounding is what it would be with q - 32 itself.
  static __device__ __forceinline__ float dot(const Regs& r, u32 c, const float (&xr)[64], const float (&sx)[NSUM]) {
    (void)sx;
    float dsc[4];
    scales(r, c, dsc);
    float s[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      u32 q[4];
      quants_s4(r, t, r.c[t] ^ 0xAAAAAAAAu, q);
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        s[g] = fmaf(sbyte(q[g], 0), xr[16 * g + 4 * t + 0], s[g]);
        s[g] = fmaf(sbyte(q[g], 1), xr[16 * g + 4 * t + 1], s[g]);
        s[g] = fmaf(sbyte(q[g], 2), xr[16 * g + 4 * t + 2], s[g]);
        s[g] = fmaf(sbyte(q[g], 3), xr[16 * g + 4 * t + 3], s[g]);
      }
    }
    float acc = (dsc[0] * 0.25f) * s[0];
#pragma unroll
    for (int g = 1; g < 4; ++g) acc = fmaf(dsc[g] * 0.25f, s[g], acc);
    return acc;
  }

  static __device__ __forceinline__ void dequant(const Regs& r, u32 c, float (&w)[64]) {
    float dsc[4];
    scales(r, c, dsc);
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      u32 q[4];
      quants(r, t, q);
#pragma unroll
      for (int g = 0; g < 4; ++g)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int qv = static_cast<int>((q[g] >> (8 * i)) & 0xFFu) - 32;
          w[16 * g + 4 * t + i] = __fmul_rn(dsc[g], static_cast<float>(qv));
        }
    }
  }
};
