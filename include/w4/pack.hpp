#pragma once

// Host side of the packed W4A16 weight format: the artifact, its quantizer, the
// element-wise dequantization step every kernel reproduces, and the FP64 GEMM
// the device results are judged against.  Same names, arguments and error
// behaviour as the reference's include/w4/pack.hpp (cited per function); the
// half type is HIP's, so this header is compiled by hipcc.
//
// Layout of a PackedW for a logical N x K row-major weight matrix:
//   groups   consecutive runs of `gs` elements along K (gs % 8 == 0; the last
//            group of a row may be short), G = ceil(K / gs) per row
//   q        N * words(K) uint32; word w of row n carries k = 8w .. 8w+7, the
//            lowest nibble first
//   scales   N * G FP16 values
//   zeros    asymmetric artifacts only: one nibble per (row, group), packed
//            along G exactly like q along K
//   value    scale * (q - z), z = 8 for symmetric artifacts

#include <hip/hip_fp16.h>

#include <algorithm>
#include <cmath>
#include <cstddef>
#include <cstdint>
#include <cstring>
#include <random>
#include <stdexcept>
#include <vector>

#if defined(__HIPCC__)
#define W4_HD __host__ __device__
#else
#define W4_HD
#endif

namespace w4 {

// packed words needed for n four-bit codes (pack.hpp:33)
W4_HD inline int words(int n) { return (n + 7) / 8; }

// pack.hpp:35-41
struct PackedW {
  int N = 0, K = 0, gs = 0, G = 0;
  bool symmetric = true;
  std::vector<uint32_t> q;
  std::vector<__half> scales;
  std::vector<uint32_t> zeros;
};

namespace detail {

inline void require(bool ok, const char* what) {
  if (!ok) throw std::invalid_argument(what);
}

// float -> FP16, round to nearest even, worked on the float's bit pattern.  The
// quantizers round double -> float -> half in two steps (as the reference
// does); going through the bits keeps an optimizer from fusing the two
// conversions into one double -> half rounding, which differs on ties.
inline __half half_rn(float f) {
  uint32_t u;
  std::memcpy(&u, &f, 4);
  const uint32_t a = u & 0x7FFFFFFFu;
  uint32_t h;
  if (a > 0x7F800000u) {
    h = 0x7E00u | ((a >> 13) & 0x3FFu);  // NaN, payload kept
  } else if (a >= 0x477FF000u) {
    h = 0x7C00u;  // 65520 and above round to infinity
  } else if (a >= 0x38800000u) {
    const uint32_t m = a - 0x38000000u;  // re-biased exponent | 23-bit mantissa
    h = (m + 0x0FFFu + ((m >> 13) & 1u)) >> 13;
  } else if (a >= 0x33000000u) {  // lands in the FP16 subnormal range
    const uint32_t man = (a & 0x7FFFFFu) | 0x800000u;
    const int shift = 126 - (int)(a >> 23);
    const uint32_t kept = man >> shift, rem = man & ((1u << shift) - 1u), mid = 1u << (shift - 1);
    h = kept + ((rem > mid || (rem == mid && (kept & 1u))) ? 1u : 0u);
  } else {
    h = 0u;
  }
  const uint16_t bits = (uint16_t)(h | ((u >> 16) & 0x8000u));
  __half out;
  std::memcpy(&out, &bits, 2);
  return out;
}

inline int nibble(const uint32_t* words_, size_t index) {
  return (int)((words_[index >> 3] >> (4 * (index & 7))) & 0xFu);
}

inline void put_nibble(uint32_t* words_, size_t index, int value) {
  words_[index >> 3] |= (uint32_t)value << (4 * (index & 7));
}

inline int clamp_code(long v) { return (int)std::max(0L, std::min(15L, v)); }

// Scale and zero-point of one group (pack.hpp:86-117).  The scale is chosen in
// double, stored as FP16, and everything downstream divides by the stored
// value.  Throws when the stored scale is not finite, or is zero for a group
// that is not.
struct GroupFit {
  __half scale;
  float scale_f;
  int zero;
};

inline GroupFit fit_group(const double* v, int len, bool symmetric, const char* range_msg) {
  double lo = v[0], hi = v[0];
  for (int i = 1; i < len; ++i) {
    lo = std::min(lo, v[i]);
    hi = std::max(hi, v[i]);
  }
  double step = 1.0;
  bool has_signal;
  if (symmetric) {
    const double amax = std::max(std::fabs(lo), std::fabs(hi));
    if (amax > 0.0) step = amax / 7.0;  // codes then stay within [1, 15]
    has_signal = (lo != 0.0) || (hi != 0.0);
  } else {
    lo = std::min(lo, 0.0);  // the code range has to contain zero, or the
    hi = std::max(hi, 0.0);  // zero-point would fall outside [0, 15]
    if (hi > lo) step = (hi - lo) / 15.0;
    has_signal = hi != lo;
  }
  GroupFit f;
  f.scale = half_rn((float)step);
  f.scale_f = __half2float(f.scale);
  require(std::isfinite(f.scale_f) && !(f.scale_f == 0.0f && has_signal), range_msg);
  f.zero = symmetric ? 8 : clamp_code(std::lround(-lo / (double)f.scale_f));
  return f;
}

// Quantize `rows` rows of length K into caller-provided, zero-initialised
// storage.  Shared by quantize() and the KV-cache quantizer.
inline void quantize_rows(const double* w, size_t rows, int K, int gs, bool symmetric,
                          uint32_t* q, __half* scales, uint32_t* zeros) {
  const int G = (K + gs - 1) / gs, wk = words(K), wg = words(G);
  for (size_t n = 0; n < rows; ++n) {
    const double* row = w + n * (size_t)K;
    for (int g = 0; g < G; ++g) {
      const int k0 = g * gs, len = std::min(gs, K - k0);
      const GroupFit f =
          fit_group(row + k0, len, symmetric, "quantize: group scale outside FP16 range");
      scales[n * (size_t)G + g] = f.scale;
      for (int k = k0; k < k0 + len; ++k)
        put_nibble(q + n * (size_t)wk, (size_t)k,
                   clamp_code(std::lround(row[k] / (double)f.scale_f) + f.zero));
      if (!symmetric) put_nibble(zeros + n * (size_t)wg, (size_t)g, f.zero);
    }
  }
}

inline bool all_finite(const std::vector<double>& v) {
  for (const double x : v)
    if (!std::isfinite(x)) return false;
  return true;
}

}  // namespace detail

// pack.hpp:43-53
inline int get_q(const PackedW& p, int n, int k) {
  return detail::nibble(p.q.data() + (size_t)n * words(p.K), (size_t)k);
}
inline int get_z(const PackedW& p, int n, int g) {
  return detail::nibble(p.zeros.data() + (size_t)n * words(p.G), (size_t)g);
}
inline int zero_point(const PackedW& p, int n, int g) { return p.symmetric ? 8 : get_z(p, n, g); }

// The dequantization step (pack.hpp:58-60): one FP32 multiply, one
// round-to-nearest-even conversion.  The kernels produce the same bits.
W4_HD inline __half dequant_one(__half s, int q, int z) {
  return __float2half_rn(__half2float(s) * (float)(q - z));
}

// pack.hpp:64-130
inline PackedW quantize(const std::vector<double>& w, int N, int K, int gs, bool symmetric) {
  detail::require(N >= 1 && K >= 1, "quantize: bad dims");
  detail::require(gs >= 8 && gs % 8 == 0, "quantize: gs must be a multiple of 8");
  detail::require(w.size() == (size_t)N * (size_t)K, "quantize: size");
  detail::require(detail::all_finite(w), "quantize: non-finite input");
  PackedW p;
  p.N = N;
  p.K = K;
  p.gs = gs;
  p.G = (K + gs - 1) / gs;
  p.symmetric = symmetric;
  p.q.assign((size_t)N * words(K), 0u);
  p.scales.assign((size_t)N * p.G, __float2half_rn(0.0f));
  if (!symmetric) p.zeros.assign((size_t)N * words(p.G), 0u);
  detail::quantize_rows(w.data(), (size_t)N, K, gs, symmetric, p.q.data(), p.scales.data(),
                        symmetric ? nullptr : p.zeros.data());
  return p;
}

// pack.hpp:134-148
inline void validate_packed(const PackedW& p) {
  using detail::require;
  require(p.N >= 1 && p.K >= 1, "packed: bad dims");
  require(p.gs >= 8 && p.gs % 8 == 0, "packed: gs must be a multiple of 8");
  require(p.G == (p.K + p.gs - 1) / p.gs, "packed: G inconsistent with K, gs");
  require(p.q.size() == (size_t)p.N * (size_t)words(p.K), "packed: q size");
  require(p.scales.size() == (size_t)p.N * (size_t)p.G, "packed: scales size");
  require(p.symmetric || p.zeros.size() == (size_t)p.N * (size_t)words(p.G), "packed: zeros size");
  require(!p.symmetric || p.zeros.empty(), "packed: symmetric carries no zeros");
}

// pack.hpp:150-161
inline std::vector<__half> dequant_all(const PackedW& p) {
  validate_packed(p);
  std::vector<__half> out((size_t)p.N * p.K);
  for (int n = 0; n < p.N; ++n)
    for (int g = 0; g < p.G; ++g) {
      const __half s = p.scales[(size_t)n * p.G + g];
      const int z = zero_point(p, n, g);
      const int k1 = std::min(p.K, (g + 1) * p.gs);
      for (int k = g * p.gs; k < k1; ++k)
        out[(size_t)n * p.K + k] = dequant_one(s, get_q(p, n, k), z);
    }
  return out;
}

// FP64 reference GEMM over the FP16 inputs the device sees (pack.hpp:166-184):
// C[m,n] = sum_k x[m,k] * w[n,k], accumulated in double in k order.
inline std::vector<double> gemm_oracle(const std::vector<__half>& x, int M, int K,
                                       const std::vector<__half>& w, int N) {
  detail::require(M >= 1 && N >= 1 && K >= 1, "gemm_oracle: bad dims");
  detail::require(x.size() == (size_t)M * (size_t)K && w.size() == (size_t)N * (size_t)K,
                  "gemm_oracle: size");
  std::vector<double> xd(x.size());
  for (size_t i = 0; i < x.size(); ++i) xd[i] = (double)__half2float(x[i]);
  std::vector<double> wrow((size_t)K), c((size_t)M * N, 0.0);
  for (int n = 0; n < N; ++n) {
    for (int k = 0; k < K; ++k) wrow[k] = (double)__half2float(w[(size_t)n * K + k]);
    for (int m = 0; m < M; ++m) {
      const double* xr = xd.data() + (size_t)m * K;
      double sum = 0.0;
      for (int k = 0; k < K; ++k) sum += xr[k] * wrow[k];
      c[(size_t)m * N + n] = sum;
    }
  }
  return c;
}

// Seeded N(0,1) test data (pack.hpp:186-200).
inline std::vector<double> normal_weights(int count, uint64_t seed) {
  std::mt19937_64 engine(seed);
  std::normal_distribution<double> gauss(0.0, 1.0);
  std::vector<double> out((size_t)count);
  std::generate(out.begin(), out.end(), [&] { return gauss(engine); });
  return out;
}

inline std::vector<__half> normal_activations(int count, uint64_t seed) {
  std::mt19937_64 engine(seed);
  std::normal_distribution<double> gauss(0.0, 1.0);
  std::vector<__half> out((size_t)count);
  std::generate(out.begin(), out.end(), [&] { return detail::half_rn((float)gauss(engine)); });
  return out;
}

}  // namespace w4
