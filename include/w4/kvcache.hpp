#pragma once

// W4 KV cache, host side: format, quantizer and the FP64 decode-attention
// reference.  Same API and error behaviour as the reference's
// include/w4/kvcache.hpp (cited per function).
//
// The cache is H independent slabs in the PackedW format with positions as
// rows (N = S) and the head dimension as the packed axis (K = D); slab h of
// every array starts at h * S * <per-row size>.  Decode attention for one query
// token per head: scores q.k_t / sqrt(D), max-subtracted softmax, weighted sum
// of the value rows.

#include <hip/hip_fp16.h>

#include <cmath>
#include <cstdint>
#include <stdexcept>
#include <vector>

#include "pack.hpp"

namespace w4::kv {

// kvcache.hpp:28-34
struct KVCacheW4 {
  int H = 0, S = 0, D = 0, gs = 0, G = 0;
  bool symmetric = true;
  std::vector<uint32_t> q_k, q_v;
  std::vector<__half> s_k, s_v;
  std::vector<uint32_t> z_k, z_v;
};

// kvcache.hpp:36-55
inline void validate_cache(const KVCacheW4& c) {
  using w4::detail::require;
  require(c.H >= 1 && c.S >= 1 && c.D >= 1, "cache: bad dims");
  require(c.gs >= 8 && c.gs % 8 == 0, "cache: gs must be a multiple of 8");
  require(c.G == (c.D + c.gs - 1) / c.gs, "cache: G inconsistent with D, gs");
  const size_t rows = (size_t)c.H * c.S;
  require(c.q_k.size() == rows * words(c.D) && c.q_v.size() == rows * words(c.D), "cache: q size");
  require(c.s_k.size() == rows * c.G && c.s_v.size() == rows * c.G, "cache: scales size");
  if (c.symmetric)
    require(c.z_k.empty() && c.z_v.empty(), "cache: symmetric carries no zeros");
  else
    require(c.z_k.size() == rows * words(c.G) && c.z_v.size() == rows * words(c.G),
            "cache: zeros size");
}

// kvcache.hpp:60-108.  k and v are H*S*D doubles, head-major then
// position-major.  Rows quantize independently, so the H slabs are simply
// H*S rows of one call into the weight quantizer's row routine; its contracts
// (non-finite input, FP16 scale range) apply unchanged.
inline KVCacheW4 quantize_cache(const std::vector<double>& k, const std::vector<double>& v,
                                int H, int S, int D, int gs, bool symmetric) {
  using w4::detail::require;
  require(H >= 1 && S >= 1 && D >= 1, "quantize_cache: bad dims");
  require(gs >= 8 && gs % 8 == 0, "quantize_cache: gs must be a multiple of 8");
  const size_t rows = (size_t)H * S;
  require(k.size() == rows * D && v.size() == rows * D, "quantize_cache: size");
  require(w4::detail::all_finite(k) && w4::detail::all_finite(v), "quantize: non-finite input");
  KVCacheW4 c;
  c.H = H;
  c.S = S;
  c.D = D;
  c.gs = gs;
  c.G = (D + gs - 1) / gs;
  c.symmetric = symmetric;
  for (auto* q : {&c.q_k, &c.q_v}) q->assign(rows * words(D), 0u);
  for (auto* s : {&c.s_k, &c.s_v}) s->assign(rows * c.G, __float2half_rn(0.0f));
  if (!symmetric)
    for (auto* z : {&c.z_k, &c.z_v}) z->assign(rows * words(c.G), 0u);
  w4::detail::quantize_rows(k.data(), rows, D, gs, symmetric, c.q_k.data(), c.s_k.data(),
                            symmetric ? nullptr : c.z_k.data());
  w4::detail::quantize_rows(v.data(), rows, D, gs, symmetric, c.q_v.data(), c.s_v.data(),
                            symmetric ? nullptr : c.z_v.data());
  return c;
}

// One head's slab as a PackedW, dequantized by the shared host routine
// (kvcache.hpp:111-135).
inline std::vector<__half> dequant_head(const KVCacheW4& c, int h, bool vside) {
  validate_cache(c);
  w4::detail::require(h >= 0 && h < c.H, "dequant_head: h");
  const size_t r0 = (size_t)h * c.S, r1 = r0 + c.S;
  const auto& q = vside ? c.q_v : c.q_k;
  const auto& s = vside ? c.s_v : c.s_k;
  const auto& z = vside ? c.z_v : c.z_k;
  PackedW p;
  p.N = c.S;
  p.K = c.D;
  p.gs = c.gs;
  p.G = c.G;
  p.symmetric = c.symmetric;
  p.q.assign(q.begin() + r0 * words(c.D), q.begin() + r1 * words(c.D));
  p.scales.assign(s.begin() + r0 * c.G, s.begin() + r1 * c.G);
  if (!c.symmetric) p.zeros.assign(z.begin() + r0 * words(c.G), z.begin() + r1 * words(c.G));
  return dequant_all(p);
}

namespace detail {

// softmax(q K^T / sqrt(D)) V for one head in double, over FP16-exact K and V
// (S x D each).  Each output element adds its terms in position order.
inline void attend_head(const __half* q, const std::vector<__half>& kd,
                        const std::vector<__half>& vd, int S, int D, double* out) {
  const double inv_sqrt_d = 1.0 / std::sqrt((double)D);
  std::vector<double> p((size_t)S), qd((size_t)D);
  for (int d = 0; d < D; ++d) qd[d] = (double)__half2float(q[d]);
  double top = -INFINITY;
  for (int t = 0; t < S; ++t) {
    double dot = 0.0;
    for (int d = 0; d < D; ++d) dot += qd[d] * (double)__half2float(kd[(size_t)t * D + d]);
    p[t] = dot * inv_sqrt_d;
    top = std::max(top, p[t]);
  }
  double denom = 0.0;
  for (int t = 0; t < S; ++t) denom += (p[t] = std::exp(p[t] - top));
  for (int t = 0; t < S; ++t) p[t] /= denom;
  for (int d = 0; d < D; ++d) {
    double sum = 0.0;
    for (int t = 0; t < S; ++t) sum += p[t] * (double)__half2float(vd[(size_t)t * D + d]);
    out[d] = sum;
  }
}

}  // namespace detail

// kvcache.hpp:141-175.  q: H*D halves; result: H*D doubles.
inline std::vector<double> attention_reference(const std::vector<__half>& q, const KVCacheW4& c) {
  validate_cache(c);
  w4::detail::require(q.size() == (size_t)c.H * c.D, "attention_reference: q size");
  std::vector<double> out((size_t)c.H * c.D, 0.0);
  for (int h = 0; h < c.H; ++h)
    detail::attend_head(q.data() + (size_t)h * c.D, dequant_head(c, h, false),
                        dequant_head(c, h, true), c.S, c.D, out.data() + (size_t)h * c.D);
  return out;
}

// Grouped-query form (not in the reference): `group` consecutive query heads
// read slab h.  Equal to attention_reference on a cache with every slab
// repeated `group` times.
inline std::vector<double> attention_reference_gqa(const std::vector<__half>& q,
                                                   const KVCacheW4& c, int group) {
  validate_cache(c);
  w4::detail::require(group >= 1 && q.size() == (size_t)c.H * group * c.D,
                      "attention_reference: q size");
  std::vector<double> out((size_t)c.H * group * c.D, 0.0);
  for (int h = 0; h < c.H; ++h) {
    const auto kd = dequant_head(c, h, false), vd = dequant_head(c, h, true);
    for (int g = 0; g < group; ++g) {
      const size_t o = ((size_t)h * group + g) * c.D;
      detail::attend_head(q.data() + o, kd, vd, c.S, c.D, out.data() + o);
    }
  }
  return out;
}

}  // namespace w4::kv
