/* CPU oracle, C restatement (TEST INFRASTRUCTURE ONLY - never linked into the product).
 *
 * Written value-by-value from the reference's per-value index arithmetic, separately from
 * the vectorised numpy restatement in oracle/kquant.py, so the two can cross-check each
 * other.  Every function cites the builder lines it follows in
 * trueno-gpu/src/kernels/quantize.rs.  Build: see oracle/Makefile (-ffp-contract=off so a
 * mul followed by a sub is never fused; the legacy decodes are inexact and depend on that).
 *
 * Pinning: same as oracle/kquant.py - decodes A and C reduce to the public GGML Q4_K/Q6_K
 * block definitions (checked in tests/test_oracle_pins.py); decode B and the legacy decodes
 * are defined by the builder calls alone and stay "parity unpinned" against the reference.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <string.h>

enum { KQ_Q4K = 4, KQ_Q5K = 5, KQ_Q6K = 6 };

static size_t sb_bytes(int fmt) { return fmt == KQ_Q4K ? 144 : fmt == KQ_Q5K ? 176 : 210; }

/* cvt.f32.f16: exact, subnormals kept (ptx/builder.rs:1241-1250). */
static float f16_to_f32(uint16_t h) {
  uint32_t sign = (uint32_t)(h >> 15) << 31;
  int e = (h >> 10) & 31;
  uint32_t m = h & 1023u;
  float v;
  if (e == 0) {
    v = ldexpf((float)m, -24);
  } else if (e == 31) {
    uint32_t bits = sign | 0x7f800000u | (m << 13);
    memcpy(&v, &bits, 4);
    return v;
  } else {
    v = ldexpf((float)(m | 1024u), e - 25);
  }
  return sign ? -v : v;
}

static uint16_t ld16(const uint8_t* p) { return (uint16_t)(p[0] | (p[1] << 8)); }

/* 12-bit contiguous field: quantize.rs:1607-1635 / :445-475 */
static void scale_min_12bit(const uint8_t* sc, unsigned j, unsigned* s, unsigned* m) {
  unsigned bit = 12u * j, b = bit / 8u, sh = bit % 8u;
  unsigned t = ((unsigned)sc[b] | ((unsigned)sc[b + 1] << 8)) >> sh;
  *s = t & 63u;
  *m = (t >> 6) & 63u;
}

/* get_scale_min_k4: quantize.rs:1306-1385 */
static void scale_min_k4(const uint8_t* sc, unsigned j, unsigned* s, unsigned* m) {
  if (j < 4) {
    *s = sc[j] & 63u;
    *m = sc[j + 4] & 63u;
  } else {
    *s = (sc[j + 4] & 0xFu) | ((unsigned)(sc[j - 4] >> 6) << 4);
    *m = (unsigned)(sc[j + 4] >> 4) | ((unsigned)(sc[j] >> 6) << 4);
  }
}

/* 4-bit quant of value i in the 64-value-chunk order: quantize.rs:1443-1466 */
static unsigned nibble_chunked(const uint8_t* qs, unsigned i) {
  unsigned chunk = i / 64u, in_chunk = i % 64u;
  unsigned byte = qs[chunk * 32u + in_chunk % 32u];
  return (byte >> (4u * (in_chunk / 32u))) & 0xFu;
}

/* one value of one super-block; policy 0 = GEMV-family (canonical), 1 = GEMM-family (legacy) */
static float dequant_one(int fmt, int policy, const uint8_t* b, unsigned i) {
  if (fmt == KQ_Q4K || fmt == KQ_Q5K) {
    float d = f16_to_f32(ld16(b)), dmin = f16_to_f32(ld16(b + 2));
    const uint8_t* sc = b + 4;
    const uint8_t* qs = b + 16;
    unsigned j = i / 32u, s, m, q;
    if (policy == 0) {
      if (fmt == KQ_Q4K) scale_min_k4(sc, j, &s, &m);       /* :1306-1385 */
      else scale_min_12bit(sc, j, &s, &m);                   /* :1607-1635 */
      q = nibble_chunked(qs, i);
      if (fmt == KQ_Q5K) q += 16u * ((b[144 + i / 8u] >> (i % 8u)) & 1u); /* :1659-1675 */
      float ds = d * (float)s;
      float scaled = ds * (float)q;
      float dm = dmin * (float)m;
      return scaled - dm;                                    /* :1468-1471, :1677-1682 */
    }
    scale_min_12bit(sc, j, &s, &m);                          /* :445-475, :727-750 */
    float inv63 = 1.0f / 63.0f;                              /* :480 */
    float sn = (float)s * inv63, mn = (float)m * inv63;
    q = (qs[i / 2u] >> (4u * (i % 2u))) & 0xFu;              /* :488-507 */
    if (fmt == KQ_Q5K) q += 16u * ((b[144 + i / 8u] >> (i % 8u)) & 1u);  /* :775-790 */
    float dsc = d * sn;
    float scaled = dsc * (float)q;
    float dmm = dmin * mn;
    return scaled - dmm;                                     /* :509-514 */
  }
  /* Q6_K */
  float d = f16_to_f32(ld16(b + 208));
  if (policy == 0) {                                         /* :1829-1923 */
    unsigned h = i / 128u, p = i % 128u, g = p / 32u, l = p % 32u, is = l / 16u;
    unsigned su = b[192 + 8u * h + is + 2u * g];
    float scale = (float)su - 256.0f * (float)(su >> 7);     /* :1857-1868 */
    unsigned qlb = b[64u * h + l + 32u * (g & 1u)];
    unsigned nib = (qlb >> (4u * (g >> 1))) & 0xFu;
    unsigned q2 = (b[128 + 32u * h + l] >> (2u * g)) & 3u;
    float qf = (float)(nib | (q2 << 4)) - 32.0f;
    float dsc = d * scale;
    return dsc * qf;
  }
  /* :1009-1064 */
  float scale = (float)b[192 + i / 16u];
  unsigned ql = (b[i / 2u] >> (4u * (i % 2u))) & 0xFu;
  unsigned q2 = (b[128 + i / 4u] >> (2u * (i % 4u))) & 3u;
  float qf = (float)(ql + 4u * q2) - 32.0f;
  float dsc = d * scale;
  return dsc * qf;
}

/* legacy "simplified" Q4_K block of q4k_gemm_fused: 18 bytes for 32 values, f16 scale at 0 (quantize.rs:237-241),
 * nibbles at 2, value i in byte i/2, low nibble for even i (:245-262); w = scale * q (:264-267) */
void kq_dequant_simplified(const uint8_t* w, size_t n_blocks, float* out) {
  for (size_t b = 0; b < n_blocks; ++b) {
    const uint8_t* p = w + b * 18u;
    float scale = f16_to_f32(ld16(p));
    for (unsigned i = 0; i < 32; ++i) {
      unsigned q = (p[2u + i / 2u] >> (4u * (i % 2u))) & 0xFu;
      out[b * 32 + i] = scale * (float)q;
    }
  }
}

/* C[m x n] = A[m x k] . W^T in fp64 on the f32 dequantised simplified weights; c[row*n + col] (:320-327) */
void kq_gemm_simplified_fp64(const uint8_t* w, const float* a, uint32_t m, uint32_t n, uint32_t k, double* c) {
  uint32_t nb = k / 32u;
  for (uint32_t col = 0; col < n; ++col)
    for (uint32_t r = 0; r < m; ++r) {
      double acc = 0.0;
      for (uint32_t b = 0; b < nb; ++b) {
        float wv[32];
        kq_dequant_simplified(w + ((size_t)col * nb + b) * 18u, 1, wv);
        for (unsigned i = 0; i < 32; ++i) acc += (double)wv[i] * (double)a[(size_t)r * k + 32u * b + i];
      }
      c[(size_t)r * n + col] = acc;
    }
}

void kq_dequant(int fmt, int policy, const uint8_t* w, size_t n_sb, float* out) {
  size_t sb = sb_bytes(fmt);
  for (size_t b = 0; b < n_sb; ++b)
    for (unsigned i = 0; i < 256; ++i) out[b * 256 + i] = dequant_one(fmt, policy, w + b * sb, i);
}

/* y[n] = sum_k W[n,k] x[k] in fp64 on the f32 dequantised weights */
void kq_gemv_fp64(int fmt, int policy, const uint8_t* w, const float* x, uint32_t k, uint32_t n, double* y) {
  size_t sb = sb_bytes(fmt), nsb = k / 256u;
  for (uint32_t r = 0; r < n; ++r) {
    double acc = 0.0;
    const uint8_t* row = w + (size_t)r * nsb * sb;           /* :1219-1224 */
    for (size_t s = 0; s < nsb; ++s)
      for (unsigned i = 0; i < 256; ++i)
        acc += (double)dequant_one(fmt, policy, row + s * sb, i) * (double)x[s * 256 + i];
    y[r] = acc;
  }
}

/* f32 in the reference's lane and summation order: quantize.rs:1412, 1482-1518 */
void kq_gemv_ref_order_f32(int fmt, const uint8_t* w, const float* x, uint32_t k, uint32_t n, float* y) {
  size_t sb = sb_bytes(fmt), nsb = k / 256u;
  for (uint32_t r = 0; r < n; ++r) {
    float acc[32];
    for (int t = 0; t < 32; ++t) acc[t] = 0.0f;
    const uint8_t* row = w + (size_t)r * nsb * sb;
    for (size_t s = 0; s < nsb; ++s)
      for (unsigned t = 0; t < 32; ++t) {
        float p = 0.0f;
        for (unsigned j = 0; j < 8; ++j) {
          unsigned i = t + 32u * j;
          p = fmaf(x[s * 256 + i], dequant_one(fmt, 0, row + s * sb, i), p);
        }
        acc[t] = acc[t] + p;
      }
    for (int step = 16; step >= 1; step >>= 1)
      for (int t = 0; t < step; ++t) acc[t] = acc[t] + acc[t + step];
    y[r] = acc[0];
  }
}

/* C[m x n] = A[m x k] . W[n x k]^T in fp64, c[row*n + col] (quantize.rs:568-574) */
void kq_gemm_fp64(int fmt, int policy, const uint8_t* w, const float* a, uint32_t m, uint32_t n, uint32_t k, double* c) {
  size_t sb = sb_bytes(fmt), nsb = k / 256u;
  for (uint32_t col = 0; col < n; ++col) {
    const uint8_t* row = w + (size_t)col * nsb * sb;
    for (uint32_t r = 0; r < m; ++r) c[(size_t)r * n + col] = 0.0;
    for (size_t s = 0; s < nsb; ++s)
      for (unsigned i = 0; i < 256; ++i) {
        double wv = (double)dequant_one(fmt, policy, row + s * sb, i);
        for (uint32_t r = 0; r < m; ++r) c[(size_t)r * n + col] += wv * (double)a[(size_t)r * k + s * 256 + i];
      }
  }
}
