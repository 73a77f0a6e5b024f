// CPU baseline for the k-quant GEMV (TEST/BENCH INFRASTRUCTURE ONLY - the reported
// "cpu_baseline" leg; never linked into the product library).
//
// The reference has no CPU k-quant path.  What a user of its CPU crate must run is:
//   1. dequantise a weight row to f32 with the GEMV-family decode
//      (trueno-gpu/src/kernels/quantize.rs:1237-1483 Q4_K, :1589-1693 Q5_K, :1806-1934 Q6_K);
//   2. Matrix::matvec semantics (src/matrix.rs:1657-1741): one dot product per row, rows
//      spread over all host threads when rows >= 4096 (the rayon path, :1676-1716);
//   3. the dot product pattern of Avx2Backend::dot (src/backends/avx2.rs:159-216): four
//      independent 8-lane FMA accumulators over 32 floats per step, an 8-wide tail into
//      accumulator 0, (a0+a1)+(a2+a3), a horizontal add, then a scalar tail; without AVX2
//      the scalar loop of src/backends/scalar.rs:66-91.
// This file restates that in C++17 with std::thread.  Block-at-a-time decode, scalar.
#include <algorithm>
#include <atomic>
#include <chrono>
#include <cstdint>
#include <cstring>
#include <thread>
#include <vector>
#if defined(__AVX2__) && defined(__FMA__)
#include <immintrin.h>
#endif

namespace {

float half_bits_to_float(uint16_t h) {
  uint32_t sign = uint32_t(h >> 15) << 31, e = (h >> 10) & 31u, m = h & 1023u, bits;
  if (e == 0) {
    if (m == 0) {
      bits = sign;
    } else {  // subnormal: renormalise
      int shift = 0;
      while (!(m & 1024u)) { m <<= 1; ++shift; }
      bits = sign | ((113u - shift) << 23) | ((m & 1023u) << 13);
    }
  } else if (e == 31) {
    bits = sign | 0x7f800000u | (m << 13);
  } else {
    bits = sign | ((e + 112u) << 23) | (m << 13);
  }
  float f;
  std::memcpy(&f, &bits, 4);
  return f;
}

inline uint16_t rd16(const uint8_t* p) { return uint16_t(p[0] | (p[1] << 8)); }

// decode A: 144-byte block -> 256 floats
void decode_q4k_block(const uint8_t* b, float* out) {
  const float d = half_bits_to_float(rd16(b)), dmin = half_bits_to_float(rd16(b + 2));
  const uint8_t* sc = b + 4;
  const uint8_t* qs = b + 16;
  for (int pair = 0; pair < 4; ++pair) {
    float ds[2], dm[2];
    for (int u = 0; u < 2; ++u) {
      int j = 2 * pair + u;
      unsigned s, m;
      if (j < 4) { s = sc[j] & 63u; m = sc[j + 4] & 63u; }
      else { s = (sc[j + 4] & 15u) | (unsigned(sc[j - 4] >> 6) << 4); m = unsigned(sc[j + 4] >> 4) | (unsigned(sc[j] >> 6) << 4); }
      ds[u] = d * float(s);
      dm[u] = dmin * float(m);
    }
    const uint8_t* q = qs + 32 * pair;
    float* o = out + 64 * pair;
    for (int l = 0; l < 32; ++l) {
      o[l] = ds[0] * float(q[l] & 15u) - dm[0];
      o[l + 32] = ds[1] * float(q[l] >> 4) - dm[1];
    }
  }
}

// decode B: 176-byte block
void decode_q5k_block(const uint8_t* b, float* out) {
  const float d = half_bits_to_float(rd16(b)), dmin = half_bits_to_float(rd16(b + 2));
  const uint8_t* sc = b + 4;
  const uint8_t* qs = b + 16;
  const uint8_t* qh = b + 144;
  for (int j = 0; j < 8; ++j) {
    unsigned bit = 12u * j, t = (unsigned(sc[bit / 8]) | (unsigned(sc[bit / 8 + 1]) << 8)) >> (bit % 8);
    const float ds = d * float(t & 63u), dm = dmin * float((t >> 6) & 63u);
    const uint8_t* q = qs + 32 * (j / 2);
    const unsigned shift = 4u * (j & 1);
    for (int l = 0; l < 32; ++l) {
      unsigned i = 32u * j + l;
      unsigned v = ((q[l] >> shift) & 15u) + 16u * ((qh[i / 8] >> (i % 8)) & 1u);
      out[i] = ds * float(v) - dm;
    }
  }
}

// decode C: 210-byte block
void decode_q6k_block(const uint8_t* b, float* out) {
  const float d = half_bits_to_float(rd16(b + 208));
  const int8_t* sc = reinterpret_cast<const int8_t*>(b + 192);
  for (int h = 0; h < 2; ++h) {
    const uint8_t* ql = b + 64 * h;
    const uint8_t* qh = b + 128 + 32 * h;
    float* o = out + 128 * h;
    for (int l = 0; l < 32; ++l) {
      int is = l / 16;
      int q0 = int((ql[l] & 15u) | (((qh[l] >> 0) & 3u) << 4)) - 32;
      int q1 = int((ql[l + 32] & 15u) | (((qh[l] >> 2) & 3u) << 4)) - 32;
      int q2 = int((ql[l] >> 4) | (((qh[l] >> 4) & 3u) << 4)) - 32;
      int q3 = int((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3u) << 4)) - 32;
      o[l] = (d * float(sc[8 * h + is])) * float(q0);
      o[l + 32] = (d * float(sc[8 * h + is + 2])) * float(q1);
      o[l + 64] = (d * float(sc[8 * h + is + 4])) * float(q2);
      o[l + 96] = (d * float(sc[8 * h + is + 6])) * float(q3);
    }
  }
}

size_t block_bytes(int fmt) { return fmt == 4 ? 144 : fmt == 5 ? 176 : 210; }

void decode_row(int fmt, const uint8_t* row, uint32_t nsb, float* out) {
  const size_t sb = block_bytes(fmt);
  for (uint32_t s = 0; s < nsb; ++s) {
    if (fmt == 4) decode_q4k_block(row + s * sb, out + 256 * s);
    else if (fmt == 5) decode_q5k_block(row + s * sb, out + 256 * s);
    else decode_q6k_block(row + s * sb, out + 256 * s);
  }
}

float dot_row(const float* a, const float* b, size_t len) {
  size_t i = 0;
  float result = 0.0f;
#if defined(__AVX2__) && defined(__FMA__)
  __m256 s0 = _mm256_setzero_ps(), s1 = s0, s2 = s0, s3 = s0;
  for (; i + 32 <= len; i += 32) {
    s0 = _mm256_fmadd_ps(_mm256_loadu_ps(a + i), _mm256_loadu_ps(b + i), s0);
    s1 = _mm256_fmadd_ps(_mm256_loadu_ps(a + i + 8), _mm256_loadu_ps(b + i + 8), s1);
    s2 = _mm256_fmadd_ps(_mm256_loadu_ps(a + i + 16), _mm256_loadu_ps(b + i + 16), s2);
    s3 = _mm256_fmadd_ps(_mm256_loadu_ps(a + i + 24), _mm256_loadu_ps(b + i + 24), s3);
  }
  for (; i + 8 <= len; i += 8) s0 = _mm256_fmadd_ps(_mm256_loadu_ps(a + i), _mm256_loadu_ps(b + i), s0);
  __m256 s = _mm256_add_ps(_mm256_add_ps(s0, s1), _mm256_add_ps(s2, s3));
  __m128 q = _mm_add_ps(_mm256_castps256_ps128(s), _mm256_extractf128_ps(s, 1));
  q = _mm_add_ps(q, _mm_movehl_ps(q, q));
  q = _mm_add_ss(q, _mm_shuffle_ps(q, q, 1));
  result = _mm_cvtss_f32(q);
#endif
  float tail = 0.0f;
  for (; i < len; ++i) tail += a[i] * b[i];
  return result + tail;
}

template <class F>
void parallel_rows(uint32_t n, int threads, F&& body) {
  // rows >= 4096 go parallel (src/matrix.rs:1676-1716); smaller matrices stay serial (:1719-1738)
  if (threads <= 1 || n < 4096) {
    body(0u, n, 0);
    return;
  }
  std::vector<std::thread> pool;
  std::atomic<uint32_t> next{0};
  const uint32_t grain = 16;
  for (int t = 0; t < threads; ++t)
    pool.emplace_back([&, t] {
      for (;;) {
        uint32_t r0 = next.fetch_add(grain);
        if (r0 >= n) break;
        body(r0, std::min(n, r0 + grain), t);
      }
    });
  for (auto& th : pool) th.join();
}

double now_s() {
  return std::chrono::duration<double>(std::chrono::steady_clock::now().time_since_epoch()).count();
}

}  // namespace

extern "C" {

int kq_cpu_threads(void) {
  unsigned n = std::thread::hardware_concurrency();
  return n ? int(n) : 1;
}

int kq_cpu_has_avx2(void) {
#if defined(__AVX2__) && defined(__FMA__)
  return 1;
#else
  return 0;
#endif
}

// one block -> 256 floats (exposed so the tests can check this third restatement too)
void kq_cpu_decode_block(int fmt, const uint8_t* block, float* out) { decode_row(fmt, block, 1, out); }

// dequantise each row to f32 then dot with x.  Returns seconds per call (mean of `reps`).
double kq_cpu_dequant_matvec(int fmt, const uint8_t* w, const float* x, uint32_t k, uint32_t n, float* y,
                             int threads, int reps) {
  const uint32_t nsb = k / 256u;
  const size_t row_bytes = size_t(nsb) * block_bytes(fmt);
  std::vector<std::vector<float>> scratch(size_t(std::max(threads, 1)), std::vector<float>(k));
  double t0 = now_s();
  for (int r = 0; r < reps; ++r)
    parallel_rows(n, threads, [&](uint32_t r0, uint32_t r1, int tid) {
      float* buf = scratch[size_t(tid)].data();
      for (uint32_t row = r0; row < r1; ++row) {
        decode_row(fmt, w + row * row_bytes, nsb, buf);
        y[row] = dot_row(buf, x, k);
      }
    });
  return (now_s() - t0) / double(std::max(reps, 1));
}

// matvec on weights already dequantised to f32 (4 bytes per weight).  Seconds per call.
double kq_cpu_matvec_f32(const float* w, const float* x, uint32_t k, uint32_t n, float* y, int threads, int reps) {
  double t0 = now_s();
  for (int r = 0; r < reps; ++r)
    parallel_rows(n, threads, [&](uint32_t r0, uint32_t r1, int) {
      for (uint32_t row = r0; row < r1; ++row) y[row] = dot_row(w + size_t(row) * k, x, k);
    });
  return (now_s() - t0) / double(std::max(reps, 1));
}

}  // extern "C"
