#pragma once

// Host side of the MXFP4 weight format (OCP microscaling): E2M1 elements with
// one E8M0 power-of-two scale per block of 32 along K.  Same API and error
// behaviour as the reference's include/w4/mx.hpp (cited per function).
//
//   q        N * words(K) uint32, 8 codes per word, lowest nibble first;
//            code = sign << 3 | magnitude index into {0, .5, 1, 1.5, 2, 3, 4, 6}
//   scales   N * B bytes, B = ceil(K / 32); byte b means 2^(b - 127); 255 (NaN)
//            is never produced
//   value    2^(byte - 127) * e2m1(code), rounded once to FP16
//
// The quantizer picks the smallest power of two that keeps the block maximum at
// or below 6 (no element saturates), clamps the exponent at -127, rejects a
// block that would need more than +127, and rounds magnitudes to the nearest
// table entry with ties going to the smaller one.

#include <hip/hip_fp16.h>

#include <cmath>
#include <cstdint>
#include <stdexcept>
#include <vector>

#include "pack.hpp"

namespace w4::mx {

constexpr int MX_BLOCK = 32;

// mx.hpp:39
constexpr float kE2M1[8] = {0.0f, 0.5f, 1.0f, 1.5f, 2.0f, 3.0f, 4.0f, 6.0f};

// mx.hpp:41-45
struct PackedWm {
  int N = 0, K = 0, B = 0;
  std::vector<uint32_t> q;
  std::vector<uint8_t> scales;
};

W4_HD inline int blocks(int K) { return (K + MX_BLOCK - 1) / MX_BLOCK; }

// The dequantization step (mx.hpp:56-63), decoded arithmetically: magnitude
// index i has exponent field i >> 1 and mantissa bit i & 1; a zero exponent
// field is the subnormal pair {0, 0.5}.
W4_HD inline __half dequant_one_mx(uint8_t se, int q) {
  const int ef = (q >> 1) & 3, mant = q & 1;
  const float mag = ef ? ldexpf((float)(2 + mant), ef - 2) : 0.5f * (float)mant;
  const float scale = ldexpf(1.0f, (int)se - 127);
  return __float2half_rn(scale * ((q & 8) ? -mag : mag));
}

inline int get_q(const PackedWm& p, int n, int k) {
  return detail::nibble(p.q.data() + (size_t)n * words(p.K), (size_t)k);
}

namespace detail_mx {

// Exponent of the block scale for a block whose largest magnitude is amax
// (mx.hpp:91-101): ceil(log2(amax / 6)), nudged up while 6 * 2^e still falls
// short of amax (log2 may land one low at exact powers of two).
inline int scale_exponent(double amax) {
  if (!(amax > 0.0)) return 0;
  int e = (int)std::ceil(std::log2(amax / 6.0));
  while (amax > 6.0 * std::ldexp(1.0, e)) ++e;
  if (e > 127) throw std::invalid_argument("quantize_mx: block scale outside E8M0 range");
  return e < -127 ? -127 : e;
}

inline int nearest_magnitude(double a) {
  int best = 0;
  for (int i = 1; i < 8; ++i)
    if (std::fabs((double)kE2M1[i] - a) < std::fabs((double)kE2M1[best] - a)) best = i;
  return best;
}

}  // namespace detail_mx

// mx.hpp:71-119
inline PackedWm quantize_mx(const std::vector<double>& w, int N, int K) {
  using w4::detail::require;
  require(N >= 1 && K >= 1, "quantize_mx: bad dims");
  require(w.size() == (size_t)N * (size_t)K, "quantize_mx: size");
  require(w4::detail::all_finite(w), "quantize_mx: non-finite input");
  PackedWm p;
  p.N = N;
  p.K = K;
  p.B = blocks(K);
  p.q.assign((size_t)N * words(K), 0u);
  p.scales.assign((size_t)N * p.B, (uint8_t)0);
  for (int n = 0; n < N; ++n) {
    const double* row = w.data() + (size_t)n * K;
    uint32_t* qrow = p.q.data() + (size_t)n * words(K);
    for (int b = 0; b < p.B; ++b) {
      const int k0 = b * MX_BLOCK, k1 = std::min(K, k0 + MX_BLOCK);
      double amax = 0.0;
      for (int k = k0; k < k1; ++k) amax = std::max(amax, std::fabs(row[k]));
      const int e = detail_mx::scale_exponent(amax);
      const double scale = std::ldexp(1.0, e);
      p.scales[(size_t)n * p.B + b] = (uint8_t)(e + 127);
      for (int k = k0; k < k1; ++k) {
        const double v = row[k] / scale;
        const int code = (std::signbit(v) ? 8 : 0) | detail_mx::nearest_magnitude(std::fabs(v));
        w4::detail::put_nibble(qrow, (size_t)k, code);
      }
    }
  }
  return p;
}

// mx.hpp:121-129
inline void validate_packed_mx(const PackedWm& p) {
  using w4::detail::require;
  require(p.N >= 1 && p.K >= 1, "packed mx: bad dims");
  require(p.B == blocks(p.K), "packed mx: B inconsistent with K");
  require(p.q.size() == (size_t)p.N * (size_t)words(p.K), "packed mx: q size");
  require(p.scales.size() == (size_t)p.N * (size_t)p.B, "packed mx: scales size");
}

// mx.hpp:131-140
inline std::vector<__half> dequant_all_mx(const PackedWm& p) {
  validate_packed_mx(p);
  std::vector<__half> out((size_t)p.N * p.K);
  for (int n = 0; n < p.N; ++n)
    for (int k = 0; k < p.K; ++k)
      out[(size_t)n * p.K + k] =
          dequant_one_mx(p.scales[(size_t)n * p.B + k / MX_BLOCK], get_q(p, n, k));
  return out;
}

}  // namespace w4::mx
