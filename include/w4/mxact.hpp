#pragma once
// MXFP8 activations: E4M3 elements under one E8M0 scale per 32 -- the
// activation operand of the W4A8 entry point (w4::gpu::gemm_mx_w4a8).
//
// No counterpart in the reference, whose kernels keep FP16 activations
// (include/w4/mxfused.cuh:166-198).  The format follows the reference's own
// MXFP4 definition (include/w4/mx.hpp:29-41, 71-119) with the element type
// exchanged: block of 32 along K, scale 2^(byte - 127), the block exponent the
// smallest e with amax <= 448 * 2^e (448 = largest E4M3 magnitude, as 6 is the
// largest E2M1 one), elements the round-to-nearest-even, saturating E4M3 code of
// float(v / 2^e) (the encoder of include/w4/kvfp8.hpp:48-53).
#include <cmath>
#include <cstdint>
#include <stdexcept>
#include <vector>

#include "kvfp8.hpp"
#include "mx.hpp"
#include "pack.hpp"

namespace w4::mxa {

constexpr int MX_BLOCK = 32;

struct PackedXm8 {
  int M = 0, K = 0, B = 0;      // B = ceil(K / 32)
  std::vector<uint8_t> q;       // M * K E4M3 bytes, row-major
  std::vector<uint8_t> scales;  // M * B E8M0 bytes
};

namespace detail {
inline int scale_exponent(double amax) {
  if (!(amax > 0.0)) return 0;
  int e = -127;
  while (e <= 127 && amax > 448.0 * std::ldexp(1.0, e)) ++e;
  if (e > 127) throw std::invalid_argument("quantize_mx8: block scale outside E8M0 range");
  return e;
}
}  // namespace detail

inline PackedXm8 quantize_mx8(const std::vector<double>& x, int M, int K) {
  using w4::detail::require;
  require(M >= 1 && K >= 1, "quantize_mx8: bad dims");
  require(x.size() == (size_t)M * (size_t)K, "quantize_mx8: size");
  require(w4::detail::all_finite(x), "quantize_mx8: non-finite input");
  PackedXm8 p;
  p.M = M;
  p.K = K;
  p.B = (K + MX_BLOCK - 1) / MX_BLOCK;
  p.q.assign((size_t)M * K, (uint8_t)0);
  p.scales.assign((size_t)M * p.B, (uint8_t)0);
  for (int m = 0; m < M; ++m) {
    const double* row = x.data() + (size_t)m * K;
    for (int b = 0; b < p.B; ++b) {
      const int k0 = b * MX_BLOCK, k1 = std::min(K, k0 + MX_BLOCK);
      double amax = 0.0;
      for (int k = k0; k < k1; ++k) amax = std::max(amax, std::fabs(row[k]));
      const int e = detail::scale_exponent(amax);
      const double scale = std::ldexp(1.0, e);
      p.scales[(size_t)m * p.B + b] = (uint8_t)(e + 127);
      for (int k = k0; k < k1; ++k)
        p.q[(size_t)m * K + k] = w4::kv8::encode_f8_e4m3_satfinite((float)(row[k] / scale));
    }
  }
  return p;
}

inline void validate_packed_mx8(const PackedXm8& p) {
  using w4::detail::require;
  require(p.M >= 1 && p.K >= 1, "packed mx8: bad dims");
  require(p.B == (p.K + MX_BLOCK - 1) / MX_BLOCK, "packed mx8: B inconsistent with K");
  require(p.q.size() == (size_t)p.M * (size_t)p.K, "packed mx8: q size");
  require(p.scales.size() == (size_t)p.M * (size_t)p.B, "packed mx8: scales size");
}

// Exact value of an element: E4M3 magnitude times a power of two (FP64 holds it).
inline double dequant_one_mx8(uint8_t scale, uint8_t code) {
  return (double)w4::kv8::decode_f8_e4m3(code) * std::ldexp(1.0, (int)scale - 127);
}

inline std::vector<double> dequant_all_mx8(const PackedXm8& p) {
  validate_packed_mx8(p);
  std::vector<double> out((size_t)p.M * p.K);
  for (int m = 0; m < p.M; ++m)
    for (int k = 0; k < p.K; ++k)
      out[(size_t)m * p.K + k] =
          dequant_one_mx8(p.scales[(size_t)m * p.B + k / MX_BLOCK], p.q[(size_t)m * p.K + k]);
  return out;
}

// FP64 reference of the W4A8 product: the activations above against MXFP4
// weights (their dequantized FP16 values widened, as gemm_oracle does).
inline std::vector<double> gemm_reference_w4a8(const PackedXm8& x, const w4::mx::PackedWm& w) {
  validate_packed_mx8(x);
  w4::detail::require(x.K == w.K, "gemm_reference_w4a8: operands disagree on K");
  const std::vector<double> xd = dequant_all_mx8(x);
  const std::vector<__half> wh = w4::mx::dequant_all_mx(w);
  std::vector<double> c((size_t)x.M * w.N);
  for (int n = 0; n < w.N; ++n)
    for (int m = 0; m < x.M; ++m) {
      double acc = 0.0;
      for (int k = 0; k < x.K; ++k)
        acc += xd[(size_t)m * x.K + k] * (double)__half2float(wh[(size_t)n * w.K + k]);
      c[(size_t)m * w.N + n] = acc;
    }
  return c;
}

}  // namespace w4::mxa
