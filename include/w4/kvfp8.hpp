#pragma once

// FP8 (OCP E4M3) KV cache, host side.  Same API and error behaviour as the
// reference's include/w4/kvfp8.hpp (cited per function).
//
// The cache has the slab structure of the W4 cache (kvcache.hpp) with one E4M3
// byte per element and one FP16 scale per (position, group of gs elements);
// E4M3 is signed, so there are no zero-points.  The quantizer sets the group
// scale to amax / 448 (nothing saturates), stores it as FP16, and rounds
// element / stored-scale to E4M3 with round-to-nearest-even and finite
// saturation.  The float -> E4M3 conversion is written out here (the reference
// takes it from the CUDA FP8 header) so that it does not depend on which FP8
// flavour a toolchain header selects.

#include <hip/hip_fp16.h>

#include <cmath>
#include <cstdint>
#include <cstring>
#include <stdexcept>
#include <vector>

#include "kvcache.hpp"
#include "pack.hpp"

namespace w4::kv8 {

// kvfp8.hpp:36-40
struct KVCacheF8 {
  int H = 0, S = 0, D = 0, gs = 0, G = 0;
  std::vector<uint8_t> q_k, q_v;
  std::vector<__half> s_k, s_v;
};

// Closed-form decode (kvfp8.hpp:42-47): exponent field 0 is the subnormal row
// m * 2^-9, otherwise (8 + m) * 2^(e - 10).  The two NaN encodings are never
// produced by the quantizer and read as +-480 here.
W4_HD inline float decode_f8_e4m3(uint8_t b) {
  const int e = (b >> 3) & 15, m = b & 7;
  const float mag = e ? ldexpf((float)(8 + m), e - 10) : ldexpf((float)m, -9);
  return (b & 0x80) ? -mag : mag;
}

// kvfp8.hpp:51-53
W4_HD inline __half dequant_one_f8(__half s, uint8_t b) {
  return __float2half_rn(__half2float(s) * decode_f8_e4m3(b));
}

// float -> OCP E4M3, round to nearest even, magnitudes at or above 448 (and
// infinities) saturate to 0x7E, NaN gives 0x7F.
inline uint8_t encode_f8_e4m3_satfinite(float x) {
  uint32_t bits;
  std::memcpy(&bits, &x, 4);
  const uint8_t sign = (uint8_t)((bits >> 24) & 0x80u);
  const float a = std::fabs(x);
  if (a != a) return (uint8_t)(sign | 0x7F);
  if (a >= 448.0f) return (uint8_t)(sign | 0x7E);
  // Quantum of the binade a falls in: 2^(floor(log2 a) - 3), never below the
  // subnormal step 2^-9.  a / quantum is exact, so one nearbyint is the rounding.
  int ex = a > 0.0f ? std::ilogb(a) : -6;
  if (ex < -6) ex = -6;
  const int steps = (int)std::nearbyint(std::ldexp(a, 3 - ex));  // 0..16
  // code = steps + 8*(ex+6): a carry to 16 steps lands on the next binade's code
  const int code = ex == -6 && steps < 8 ? steps : (ex + 7) * 8 + (steps - 8);
  return (uint8_t)(sign | (code > 0x7E ? 0x7E : code));
}

// kvfp8.hpp:55-68
inline void validate_cache_f8(const KVCacheF8& c) {
  using w4::detail::require;
  require(c.H >= 1 && c.S >= 1 && c.D >= 1, "cache f8: bad dims");
  require(c.gs >= 8 && c.gs % 8 == 0, "cache f8: gs must be a multiple of 8");
  require(c.G == (c.D + c.gs - 1) / c.gs, "cache f8: G inconsistent with D, gs");
  const size_t rows = (size_t)c.H * c.S;
  require(c.q_k.size() == rows * c.D && c.q_v.size() == rows * c.D, "cache f8: q size");
  require(c.s_k.size() == rows * c.G && c.s_v.size() == rows * c.G, "cache f8: scales size");
}

// kvfp8.hpp:70-128
inline KVCacheF8 quantize_cache_f8(const std::vector<double>& k, const std::vector<double>& v,
                                   int H, int S, int D, int gs) {
  using w4::detail::require;
  require(H >= 1 && S >= 1 && D >= 1, "quantize_cache_f8: bad dims");
  require(gs >= 8 && gs % 8 == 0, "quantize_cache_f8: gs must be a multiple of 8");
  const size_t rows = (size_t)H * S;
  require(k.size() == rows * D && v.size() == rows * D, "quantize_cache_f8: size");
  require(w4::detail::all_finite(k) && w4::detail::all_finite(v),
          "quantize_cache_f8: non-finite input");
  KVCacheF8 c;
  c.H = H;
  c.S = S;
  c.D = D;
  c.gs = gs;
  c.G = (D + gs - 1) / gs;
  auto one_side = [&](const std::vector<double>& src, std::vector<uint8_t>& codes,
                      std::vector<__half>& scales) {
    codes.assign(rows * D, (uint8_t)0);
    scales.assign(rows * c.G, __float2half_rn(0.0f));
    for (size_t r = 0; r < rows; ++r)
      for (int g = 0; g < c.G; ++g) {
        const int d0 = g * gs, d1 = std::min(D, d0 + gs);
        double amax = 0.0;
        for (int d = d0; d < d1; ++d) amax = std::max(amax, std::fabs(src[r * D + d]));
        const __half sh = w4::detail::half_rn((float)(amax > 0.0 ? amax / 448.0 : 1.0));
        const float sf = __half2float(sh);
        require(std::isfinite(sf) && !(sf == 0.0f && amax > 0.0),
                "quantize_cache_f8: group scale outside FP16 range");
        scales[r * c.G + g] = sh;
        for (int d = d0; d < d1; ++d)
          codes[r * D + d] = encode_f8_e4m3_satfinite((float)(src[r * D + d] / (double)sf));
      }
  };
  one_side(k, c.q_k, c.s_k);
  one_side(v, c.q_v, c.s_v);
  return c;
}

// kvfp8.hpp:131-146
inline std::vector<__half> dequant_head_f8(const KVCacheF8& c, int h, bool vside) {
  validate_cache_f8(c);
  w4::detail::require(h >= 0 && h < c.H, "dequant_head_f8: h");
  const uint8_t* q = (vside ? c.q_v : c.q_k).data() + (size_t)h * c.S * c.D;
  const __half* s = (vside ? c.s_v : c.s_k).data() + (size_t)h * c.S * c.G;
  std::vector<__half> out((size_t)c.S * c.D);
  for (int t = 0; t < c.S; ++t)
    for (int d = 0; d < c.D; ++d)
      out[(size_t)t * c.D + d] = dequant_one_f8(s[(size_t)t * c.G + d / c.gs], q[(size_t)t * c.D + d]);
  return out;
}

// kvfp8.hpp:150-184: the FP64 reference of kvcache.hpp over the FP8 cache.
inline std::vector<double> attention_reference_f8(const std::vector<__half>& q,
                                                  const KVCacheF8& c) {
  validate_cache_f8(c);
  w4::detail::require(q.size() == (size_t)c.H * c.D, "attention_reference_f8: q size");
  std::vector<double> out((size_t)c.H * c.D, 0.0);
  for (int h = 0; h < c.H; ++h)
    w4::kv::detail::attend_head(q.data() + (size_t)h * c.D, dequant_head_f8(c, h, false),
                                dequant_head_f8(c, h, true), c.S, c.D,
                                out.data() + (size_t)h * c.D);
  return out;
}

}  // namespace w4::kv8
