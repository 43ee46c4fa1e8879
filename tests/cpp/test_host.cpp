// Host gates for the C++ headers under include/w4/ (CPU only).  Two kinds of
// check per format:
//   * the reference host suite's gates (tests/test_oracle.cpp): per-element
//     quantizer bounds on its seeded configs, hand pins, degenerate inputs and
//     the std::invalid_argument list;
//   * byte-for-byte agreement of every quantizer / dequantizer / FP64 reference
//     with the independent C oracle (oracle/w4_oracle.c) on the same inputs.
#include <cmath>
#include <cstring>
#include <vector>

#include "../../oracle/w4_oracle.h"
#include "check.hpp"
#include "w4/kvcache.hpp"
#include "w4/kvfp8.hpp"
#include "w4/kvpaged.hpp"
#include "w4/mx.hpp"
#include "w4/mxact.hpp"
#include "w4/pack.hpp"

namespace {

template <class T>
bool same_bytes(const std::vector<T>& a, const void* b, size_t n) {
  return a.size() == n && (n == 0 || std::memcmp(a.data(), b, n * sizeof(T)) == 0);
}

struct Shape { int M, N, K, gs; };
const Shape kShapes[] = {{1, 64, 64, 8},   {8, 128, 96, 16}, {16, 256, 100, 32}, {4, 96, 72, 48},
                         {2, 32, 128, 64}, {3, 40, 256, 128}, {5, 72, 40, 8}};

void w4_gates(Checks& t) {
  for (const bool sym : {true, false})
    for (size_t i = 0; i < sizeof kShapes / sizeof *kShapes; ++i) {
      const Shape c = kShapes[i];
      const uint64_t seed = 0x44A1ULL ^ (uint64_t)(i * 977 + (sym ? 0 : 1));
      const auto w = w4::normal_weights(c.N * c.K, seed);
      // the generators themselves
      std::vector<double> wo(w.size());
      orc_normal_weights(wo.data(), wo.size(), seed);
      t.expect(wo == w, "normal_weights stream");
      const auto p = w4::quantize(w, c.N, c.K, c.gs, sym);
      const auto wd = w4::dequant_all(p);
      bool in_bounds = true;
      for (int n = 0; n < c.N; ++n)
        for (int k = 0; k < c.K; ++k) {
          const double sf = __half2float(p.scales[(size_t)n * p.G + k / p.gs]);
          const int q = w4::get_q(p, n, k);
          const double tol = ((q == 0 || q == 15) ? 1.1 : 0.52) * sf + 1e-12;
          in_bounds &= std::fabs((double)__half2float(wd[(size_t)n * c.K + k]) - w[(size_t)n * c.K + k]) <= tol;
        }
      t.expect(in_bounds, "w4 per-element bound");
      // oracle agreement
      std::vector<uint32_t> oq(p.q.size()), oz(sym ? 0 : p.zeros.size());
      std::vector<uint16_t> os(p.scales.size()), ow(wd.size());
      t.expect(orc_quantize(w.data(), w.size(), c.N, c.K, c.gs, sym, oq.data(), os.data(),
                            sym ? nullptr : oz.data()) == 0, "oracle quantize runs");
      t.expect(same_bytes(p.q, oq.data(), oq.size()), "quantize codes == oracle");
      t.expect(same_bytes(p.scales, os.data(), os.size()), "quantize scales == oracle");
      t.expect(sym ? p.zeros.empty() : same_bytes(p.zeros, oz.data(), oz.size()), "quantize zeros == oracle");
      orc_dequant_all(c.N, c.K, c.gs, p.G, sym, oq.data(), oq.size(), os.data(), os.size(),
                      sym ? nullptr : oz.data(), oz.size(), ow.data());
      t.expect(same_bytes(wd, ow.data(), ow.size()), "dequant_all == oracle");
      const auto x = w4::normal_activations(c.M * c.K, seed + 1);
      std::vector<uint16_t> ox(x.size());
      orc_normal_activations(ox.data(), ox.size(), seed + 1);
      t.expect(same_bytes(x, ox.data(), ox.size()), "normal_activations stream");
      const auto ref = w4::gemm_oracle(x, c.M, c.K, wd, c.N);
      std::vector<double> oref(ref.size());
      orc_gemm_oracle(ox.data(), ox.size(), c.M, c.K, ow.data(), ow.size(), c.N, oref.data());
      t.expect(ref == oref, "gemm_oracle == oracle, bit for bit");
    }
  {  // x = [1,2], W = [[3,4],[5,6]] -> [11,17]
    const std::vector<__half> x = {__float2half_rn(1.f), __float2half_rn(2.f)};
    const std::vector<__half> w = {__float2half_rn(3.f), __float2half_rn(4.f), __float2half_rn(5.f),
                                   __float2half_rn(6.f)};
    const auto c = w4::gemm_oracle(x, 1, 2, w, 2);
    t.expect(c[0] == 11.0 && c[1] == 17.0, "gemm_oracle hand pin");
  }
  for (const bool sym : {true, false}) {
    const auto p = w4::quantize(std::vector<double>(64 * 64, 0.0), 64, 64, 32, sym);
    bool zero = true, unit = true;
    for (const auto& v : w4::dequant_all(p)) zero &= __half2float(v) == 0.0f;
    for (const auto& s : p.scales) unit &= __half2float(s) == 1.0f;
    t.expect(zero && unit, "all-zero groups: scale 1, exact zeros");
  }
  const std::vector<double> ok(64 * 64, 0.5);
  t.throws_invalid([&] { w4::quantize(ok, 0, 64, 8, true); }, "N=0");
  t.throws_invalid([&] { w4::quantize(ok, 64, 64, 0, true); }, "gs=0");
  t.throws_invalid([&] { w4::quantize(ok, 64, 64, 7, true); }, "gs=7");
  t.throws_invalid([&] { w4::quantize(ok, 64, 64, 9, true); }, "gs=9");
  t.throws_invalid([&] { w4::quantize(std::vector<double>(10, 0.0), 64, 64, 8, true); }, "size mismatch");
  for (const bool sym : {true, false}) {
    auto bad = ok;
    bad[3] = std::nan("");
    t.throws_invalid([&] { w4::quantize(bad, 64, 64, 8, sym); }, "NaN");
    bad[3] = INFINITY;
    t.throws_invalid([&] { w4::quantize(bad, 64, 64, 8, sym); }, "inf");
    bad[3] = 1e300;
    t.throws_invalid([&] { w4::quantize(bad, 64, 64, 8, sym); }, "scale overflows FP16");
    t.throws_invalid([&] { w4::quantize(std::vector<double>(64 * 64, 1e-12), 64, 64, 8, sym); },
                     "scale underflows FP16");
  }
  auto p = w4::quantize(ok, 64, 64, 8, true);
  auto bad_gs = p;
  bad_gs.gs = 7;
  t.throws_invalid([&] { w4::dequant_all(bad_gs); }, "dequant gs=7");
  auto bad_sizes = p;
  bad_sizes.q.resize(3);
  t.throws_invalid([&] { w4::dequant_all(bad_sizes); }, "dequant q size");
  auto sym_zeros = p;
  sym_zeros.zeros.resize(8);
  t.throws_invalid([&] { w4::dequant_all(sym_zeros); }, "symmetric with zeros");
  t.throws_invalid([&] { w4::gemm_oracle(std::vector<__half>(3), 2, 2, std::vector<__half>(4), 1); },
                   "oracle size mismatch");
  {  // the header's float -> half rounding, against the oracle's, on a dense sweep
    bool conv_ok = true;
    for (uint64_t i = 0; i < (1ull << 32); i += 257) {
      const uint32_t b = (uint32_t)i;
      float f;
      std::memcpy(&f, &b, 4);
      if (f != f) continue;
      const __half hv = w4::detail::half_rn(f);
      uint16_t hb;
      std::memcpy(&hb, &hv, 2);
      conv_ok &= hb == orc_f32_to_f16(f);
    }
    t.expect(conv_ok, "half_rn == oracle float->half");
  }
  // dequant_one over every scale bit pattern and code difference
  bool step_ok = true;
  for (uint32_t s = 0; s < 65536; ++s) {
    const uint16_t sb = (uint16_t)s;
    __half sh;
    std::memcpy(&sh, &sb, 2);
    if (__half2float(sh) != __half2float(sh)) continue;  // NaN scales are not artifacts
    for (int d = -15; d <= 15; ++d) {
      const __half got = w4::dequant_one(sh, d > 0 ? d : 0, d > 0 ? 0 : -d);
      uint16_t gb;
      std::memcpy(&gb, &got, 2);
      step_ok &= gb == orc_dequant_one(sb, d > 0 ? d : 0, d > 0 ? 0 : -d);
    }
  }
  t.expect(step_ok, "dequant_one == oracle on every (scale, q - z)");
}

void mx_gates(Checks& t) {
  const int shapes[][2] = {{64, 64}, {128, 96}, {256, 100}, {96, 72}, {32, 33}, {40, 256}, {72, 40}};
  for (size_t i = 0; i < 7; ++i) {
    const int N = shapes[i][0], K = shapes[i][1];
    const auto w = w4::normal_weights(N * K, 0x9E4FULL ^ (uint64_t)(i * 977));
    const auto p = w4::mx::quantize_mx(w, N, K);
    const auto wd = w4::mx::dequant_all_mx(p);
    bool in_bounds = true, unsat = true;
    for (int n = 0; n < N; ++n)
      for (int k = 0; k < K; ++k) {
        const double s = std::ldexp(1.0, (int)p.scales[(size_t)n * p.B + k / 32] - 127);
        const int idx = w4::mx::get_q(p, n, k) & 7;
        const double left = idx > 0 ? w4::mx::kE2M1[idx] - w4::mx::kE2M1[idx - 1] : 0.5;
        const double right = idx < 7 ? w4::mx::kE2M1[idx + 1] - w4::mx::kE2M1[idx] : left;
        in_bounds &= std::fabs((double)__half2float(wd[(size_t)n * K + k]) - w[(size_t)n * K + k]) <=
                     0.5 * std::max(left, right) * s + 1e-12;
      }
    for (int n = 0; n < N; ++n)
      for (int b = 0; b < p.B; ++b) {
        double amax = 0.0;
        for (int k = b * 32; k < std::min(K, b * 32 + 32); ++k) amax = std::max(amax, std::fabs(w[(size_t)n * K + k]));
        unsat &= amax <= 6.0 * std::ldexp(1.0, (int)p.scales[(size_t)n * p.B + b] - 127) * (1.0 + 1e-12);
      }
    t.expect(in_bounds, "mx per-element bound");
    t.expect(unsat, "mx no block saturates");
    std::vector<uint32_t> oq(p.q.size());
    std::vector<uint8_t> os(p.scales.size());
    std::vector<uint16_t> ow(wd.size());
    orc_quantize_mx(w.data(), w.size(), N, K, oq.data(), os.data());
    orc_dequant_all_mx(N, K, p.B, oq.data(), oq.size(), os.data(), os.size(), ow.data());
    t.expect(same_bytes(p.q, oq.data(), oq.size()) && same_bytes(p.scales, os.data(), os.size()),
             "quantize_mx == oracle");
    t.expect(same_bytes(wd, ow.data(), ow.size()), "dequant_all_mx == oracle");
  }
  {
    const auto p = w4::mx::quantize_mx(std::vector<double>(64, 3.0), 2, 32);
    const auto wd = w4::mx::dequant_all_mx(p);
    t.expect(p.scales[0] == 126 && p.scales[1] == 126, "mx pin: scale byte 126");
    t.expect(__half2float(wd[0]) == 3.0f && __half2float(wd[63]) == 3.0f, "mx pin: exact 3.0");
    t.expect(w4::mx::get_q(p, 0, 0) == 7, "mx pin: code 7");
  }
  {
    const auto p = w4::mx::quantize_mx(std::vector<double>(32, -2.0), 1, 32);
    t.expect(__half2float(w4::mx::dequant_all_mx(p)[0]) == -2.0f && (w4::mx::get_q(p, 0, 0) & 8), "mx sign");
  }
  {
    const auto p = w4::mx::quantize_mx(std::vector<double>(64 * 64, 0.0), 64, 64);
    bool zero = true;
    for (const auto& v : w4::mx::dequant_all_mx(p)) zero &= __half2float(v) == 0.0f;
    t.expect(zero && p.scales[0] == 127, "mx all-zero input");
  }
  bool step_ok = true;
  for (int se = 0; se < 255; ++se)
    for (int q = 0; q < 16; ++q) {
      const __half got = w4::mx::dequant_one_mx((uint8_t)se, q);
      uint16_t gb;
      std::memcpy(&gb, &got, 2);
      step_ok &= gb == orc_dequant_one_mx((uint8_t)se, q);
    }
  t.expect(step_ok, "dequant_one_mx == oracle on every (scale byte, code)");
  const std::vector<double> ok(64 * 64, 0.5);
  t.throws_invalid([&] { w4::mx::quantize_mx(ok, 0, 64); }, "mx N=0");
  t.throws_invalid([&] { w4::mx::quantize_mx(std::vector<double>(10), 64, 64); }, "mx size");
  auto bad = ok;
  bad[3] = std::nan("");
  t.throws_invalid([&] { w4::mx::quantize_mx(bad, 64, 64); }, "mx NaN");
  bad[3] = 1e300;
  t.throws_invalid([&] { w4::mx::quantize_mx(bad, 64, 64); }, "mx scale overflow");
  auto p = w4::mx::quantize_mx(ok, 64, 64);
  p.q.resize(3);
  t.throws_invalid([&] { w4::mx::dequant_all_mx(p); }, "mx dequant size");
}

void kv_gates(Checks& t) {
  for (const bool sym : {true, false}) {
    const int H = 3, S = 5, D = 24, gs = 8;
    const auto k = w4::normal_weights(H * S * D, 0xC1U), v = w4::normal_weights(H * S * D, 0xC2U);
    const auto c = w4::kv::quantize_cache(k, v, H, S, D, gs, sym);
    for (int h = 0; h < H; ++h) {
      const auto alone = w4::dequant_all(w4::quantize(
          std::vector<double>(k.begin() + (size_t)h * S * D, k.begin() + (size_t)(h + 1) * S * D), S, D, gs, sym));
      const auto slab = w4::kv::dequant_head(c, h, false);
      t.expect(same_bytes(alone, slab.data(), slab.size()), "cache slab == per-head quantize");
    }
    // FP64 attention == oracle
    const auto q = w4::normal_activations(H * D, 0xC3U);
    const auto ref = w4::kv::attention_reference(q, c);
    std::vector<uint16_t> k16((size_t)H * S * D), v16(k16.size());
    for (int h = 0; h < H; ++h) {
      const auto kh = w4::kv::dequant_head(c, h, false), vh = w4::kv::dequant_head(c, h, true);
      std::memcpy(k16.data() + (size_t)h * S * D, kh.data(), kh.size() * 2);
      std::memcpy(v16.data() + (size_t)h * S * D, vh.data(), vh.size() * 2);
    }
    std::vector<double> oref(ref.size());
    orc_attention_f16((const uint16_t*)q.data(), k16.data(), v16.data(), H, 1, S, D, oref.data());
    t.expect(ref == oref, "attention_reference == oracle, bit for bit");
  }
  {  // zero keys: uniform softmax, output is the mean of the two V rows
    const int D = 8;
    std::vector<double> k(2 * D, 0.0), v(2 * D, 0.0);
    for (int d = 0; d < D; ++d) v[d] = 1.0, v[D + d] = 3.0;
    const auto c = w4::kv::quantize_cache(k, v, 1, 2, D, 8, true);
    const auto vd = w4::kv::dequant_head(c, 0, true);
    const auto out = w4::kv::attention_reference(std::vector<__half>(D, __float2half_rn(1.0f)), c);
    bool ok = true;
    for (int d = 0; d < D; ++d)
      ok &= out[d] == 0.5 * (double)__half2float(vd[d]) + 0.5 * (double)__half2float(vd[D + d]);
    t.expect(ok, "attention pin: zero keys -> mean of V");
  }
  {  // scores near 3e4 stay finite
    const auto c = w4::kv::quantize_cache(std::vector<double>(16, 100.0), std::vector<double>(16, 0.5), 1, 2, 8, 8, true);
    const auto out = w4::kv::attention_reference(std::vector<__half>(8, __float2half_rn(100.0f)), c);
    t.expect(std::isfinite(out[0]) && out[0] == (double)__half2float(w4::kv::dequant_head(c, 0, true)[0]),
             "attention softmax stability");
  }
  const std::vector<double> ok(4 * 8, 0.5);
  t.throws_invalid([&] { w4::kv::quantize_cache(ok, ok, 0, 4, 8, 8, true); }, "kv H=0");
  t.throws_invalid([&] { w4::kv::quantize_cache(ok, ok, 1, 4, 8, 7, true); }, "kv gs=7");
  t.throws_invalid([&] { w4::kv::quantize_cache(ok, ok, 1, 4, 8, 0, true); }, "kv gs=0");
  t.throws_invalid([&] { w4::kv::quantize_cache(std::vector<double>(10), ok, 1, 4, 8, 8, true); }, "kv size");
  auto c = w4::kv::quantize_cache(ok, ok, 1, 4, 8, 8, true);
  auto bad = c;
  bad.G = 2;
  t.throws_invalid([&] { w4::kv::dequant_head(bad, 0, false); }, "kv G inconsistent");
  t.throws_invalid([&] { w4::kv::dequant_head(c, 1, false); }, "kv h out of range");
  t.throws_invalid([&] { w4::kv::attention_reference(std::vector<__half>(3), c); }, "kv q size");
}

void f8_gates(Checks& t) {
  bool enc_ok = true, dec_ok = true;
  for (int b = 0; b < 256; ++b) dec_ok &= w4::kv8::decode_f8_e4m3((uint8_t)b) == orc_decode_f8_e4m3((uint8_t)b);
  for (uint32_t i = 0; i < (1u << 22); ++i) {  // a dense sweep of float bit patterns
    const uint32_t bits = i * 1021u + 12345u;
    float x;
    std::memcpy(&x, &bits, 4);
    enc_ok &= w4::kv8::encode_f8_e4m3_satfinite(x) == orc_f32_to_e4m3_satfinite(x);
  }
  for (int b = 0; b < 0x7F; ++b) {  // every value is a fixed point
    const float vpos = w4::kv8::decode_f8_e4m3((uint8_t)b);
    enc_ok &= w4::kv8::encode_f8_e4m3_satfinite(vpos) == b;
    enc_ok &= w4::kv8::encode_f8_e4m3_satfinite(-vpos) == (b | 0x80);
  }
  t.expect(dec_ok, "decode_f8_e4m3 == oracle");
  t.expect(enc_ok, "E4M3 encode == oracle, fixed points");
  const int shapes[][2] = {{64, 64}, {7, 96}, {16, 100}, {5, 40}, {3, 72}};
  for (size_t i = 0; i < 5; ++i) {
    const int S = shapes[i][0], D = shapes[i][1];
    const uint64_t seed = 0x8F1DULL ^ (uint64_t)(i * 977);
    const auto k = w4::normal_weights(S * D, seed), v = w4::normal_weights(S * D, seed + 1);
    const auto c = w4::kv8::quantize_cache_f8(k, v, 1, S, D, 32);
    std::vector<uint8_t> ok8(c.q_k.size()), ov8(c.q_v.size());
    std::vector<uint16_t> osk(c.s_k.size()), osv(c.s_v.size()), ow((size_t)S * D);
    orc_quantize_cache_f8(k.data(), k.size(), v.data(), v.size(), 1, S, D, 32, ok8.data(), osk.data(),
                          ov8.data(), osv.data());
    t.expect(c.q_k == ok8 && c.q_v == ov8, "quantize_cache_f8 codes == oracle");
    t.expect(same_bytes(c.s_k, osk.data(), osk.size()) && same_bytes(c.s_v, osv.data(), osv.size()),
             "quantize_cache_f8 scales == oracle");
    orc_dequant_f8(ov8.data(), osv.data(), S, D, 32, ow.data());
    const auto wd = w4::kv8::dequant_head_f8(c, 0, true);
    t.expect(same_bytes(wd, ow.data(), ow.size()), "dequant_head_f8 == oracle");
    bool unsat = true;
    for (int r = 0; r < S; ++r)
      for (int g = 0; g < c.G; ++g) {
        double amax = 0.0;
        for (int d = g * 32; d < std::min(D, g * 32 + 32); ++d) amax = std::max(amax, std::fabs(k[(size_t)r * D + d]));
        unsat &= amax <= 448.0 * (double)__half2float(c.s_k[(size_t)r * c.G + g]) * (1.0 + 1e-3);
      }
    t.expect(unsat, "f8 no group saturates");
  }
  {
    const std::vector<double> w(64, 1.0);
    const auto c = w4::kv8::quantize_cache_f8(w, w, 1, 8, 8, 8);
    t.expect(c.q_k[0] == 0x7E && __half2float(w4::kv8::dequant_head_f8(c, 0, false)[0]) == 1.0f, "f8 pin 0x7E");
    const std::vector<double> n(64, -2.0);
    const auto c2 = w4::kv8::quantize_cache_f8(n, n, 1, 8, 8, 8);
    t.expect((c2.q_v[0] & 0x80) && __half2float(w4::kv8::dequant_head_f8(c2, 0, true)[0]) == -2.0f, "f8 sign");
  }
  const std::vector<double> ok(4 * 8, 0.5);
  t.throws_invalid([&] { w4::kv8::quantize_cache_f8(ok, ok, 0, 4, 8, 8); }, "f8 H=0");
  t.throws_invalid([&] { w4::kv8::quantize_cache_f8(ok, ok, 1, 4, 8, 0); }, "f8 gs=0");
  t.throws_invalid([&] { w4::kv8::quantize_cache_f8(ok, ok, 1, 4, 8, 7); }, "f8 gs=7");
  t.throws_invalid([&] { w4::kv8::quantize_cache_f8(std::vector<double>(10), ok, 1, 4, 8, 8); }, "f8 size");
  auto bad = ok;
  bad[3] = std::nan("");
  t.throws_invalid([&] { w4::kv8::quantize_cache_f8(bad, ok, 1, 4, 8, 8); }, "f8 NaN");
  bad[3] = 1e300;
  t.throws_invalid([&] { w4::kv8::quantize_cache_f8(bad, ok, 1, 4, 8, 8); }, "f8 scale overflow");
  t.throws_invalid([&] { w4::kv8::quantize_cache_f8(std::vector<double>(4 * 8, 1e-8), ok, 1, 4, 8, 8); },
                   "f8 scale underflow");
  auto c = w4::kv8::quantize_cache_f8(ok, ok, 1, 4, 8, 8);
  t.throws_invalid([&] { w4::kv8::dequant_head_f8(c, 1, false); }, "f8 h out of range");
  t.throws_invalid([&] { w4::kv8::attention_reference_f8(std::vector<__half>(3), c); }, "f8 q size");
}

void paged_gates(Checks& t) {
  const auto k = w4::normal_weights(2 * 37 * 24, 0x7A11), v = w4::normal_weights(2 * 37 * 24, 0x7A12);
  const auto cc = w4::kv::quantize_cache(k, v, 2, 37, 24, 8, true);
  const int page = 16, npages = 3, wd = w4::words(24);
  const std::vector<int> bt = {2, 0, 1};
  const auto pc = w4::kv::paged_from_contiguous(cc, page, bt);
  w4::kv::validate_paged(pc);
  bool same = true;
  for (int h = 0; h < 2; ++h)
    for (int tt = 0; tt < 37; ++tt) {
      const size_t row = (size_t)h * npages * page + (size_t)bt[tt / page] * page + tt % page;
      same &= std::memcmp(&pc.q_k[row * wd], &cc.q_k[((size_t)h * 37 + tt) * wd], wd * 4) == 0;
      same &= std::memcmp(&pc.s_v[row * cc.G], &cc.s_v[((size_t)h * 37 + tt) * cc.G], cc.G * 2) == 0;
    }
  t.expect(same, "paged rows resolve to contiguous rows");
  t.throws_invalid([&] { w4::kv::paged_from_contiguous(cc, 0, bt); }, "paged page=0");
  t.throws_invalid([&] { w4::kv::paged_from_contiguous(cc, 16, {0, 1}); }, "paged short table");
  t.throws_invalid([&] { w4::kv::paged_from_contiguous(cc, 16, {0, 1, 1}); }, "paged repeated page");
  t.throws_invalid([&] { w4::kv::paged_from_contiguous(cc, 16, {0, 1, 9}); }, "paged entry out of pool");
  auto badpool = pc;
  badpool.q_k.resize(3);
  t.throws_invalid([&] { w4::kv::validate_paged(badpool); }, "paged q size");
}

// MXFP8 activations (additive format): the header against the C oracle byte for
// byte, per-element error bound of a 3-bit mantissa, no block saturates, exact
// round trip of representable values, contracts.
void mx8_gates(Checks& t) {
  const int shapes[][2] = {{4, 64}, {7, 100}, {3, 33}, {16, 256}, {1, 1}};
  for (size_t i = 0; i < 5; ++i) {
    const int M = shapes[i][0], K = shapes[i][1];
    auto x = w4::normal_weights(M * K, 0x8A8AULL ^ (uint64_t)(i * 131));
    for (size_t j = 0; j < x.size(); j += 5) x[j] *= 50.0;  // spread the block maxima
    const auto p = w4::mxa::quantize_mx8(x, M, K);
    std::vector<uint8_t> oq(p.q.size()), os(p.scales.size());
    t.expect(orc_quantize_mx8(x.data(), x.size(), M, K, oq.data(), os.data()) == 0 && oq == p.q &&
                 os == p.scales,
             "mx8: header == oracle bytes");
    const auto d = w4::mxa::dequant_all_mx8(p);
    std::vector<double> od(d.size());
    orc_dequant_mx8(M, K, oq.data(), os.data(), od.data());
    t.expect(od == d, "mx8: dequant header == oracle");
    bool bound = true, unsat = true;
    for (int m = 0; m < M; ++m)
      for (int k = 0; k < K; ++k) {
        const double s = std::ldexp(1.0, (int)p.scales[(size_t)m * p.B + k / 32] - 127);
        const double v = x[(size_t)m * K + k], err = std::fabs(d[(size_t)m * K + k] - v);
        // half a step of the binade of |v| / s (3 mantissa bits), or of the subnormal row
        const double step = std::max(std::ldexp(1.0, std::ilogb(std::max(std::fabs(v) / s, 1e-300)) - 3), std::ldexp(1.0, -9));
        bound &= err <= 0.5 * step * s * (1 + 1e-9);
        unsat &= std::fabs(v) <= 448.0 * s;
      }
    t.expect(bound, "mx8 per-element bound");
    t.expect(unsat, "mx8 no block saturates");
    // representable values come back exactly
    const auto p2 = w4::mxa::quantize_mx8(d, M, K);
    t.expect(w4::mxa::dequant_all_mx8(p2) == d, "mx8 round trip of representable values");
  }
  {  // block maxima on and around 448 * 2^e
    std::vector<double> x(3 * 32, 0.01);
    x[0] = 448.0; x[32] = std::nextafter(448.0, 1e9); x[64] = std::nextafter(448.0, 0.0);
    const auto p = w4::mxa::quantize_mx8(x, 3, 32);
    t.expect(p.scales[0] == 127 && p.scales[1] == 128 && p.scales[2] == 127, "mx8 scale boundaries");
    t.expect(p.q[0] == 0x7E && p.q[32] == 0x76 && p.q[64] == 0x7E, "mx8 codes at the boundaries");
  }
  t.throws_invalid([] { w4::mxa::quantize_mx8(std::vector<double>(4, 1.0), 0, 4); }, "quantize_mx8: bad dims");
  t.throws_invalid([] { w4::mxa::quantize_mx8(std::vector<double>(5, 1.0), 1, 4); }, "quantize_mx8: size");
  t.throws_invalid([] { w4::mxa::quantize_mx8(std::vector<double>(4, std::nan("")), 1, 4); },
                   "quantize_mx8: non-finite input");
  t.throws_invalid([] { w4::mxa::quantize_mx8(std::vector<double>(4, 1e300), 1, 4); },
                   "quantize_mx8: block scale outside E8M0 range");
}

}  // namespace

int main() {
  Checks t;
  mx8_gates(t);
  w4_gates(t);
  mx_gates(t);
  kv_gates(t);
  f8_gates(t);
  paged_gates(t);
  return t.finish("host");
}
