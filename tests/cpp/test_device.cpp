// Device gates through the C++ API (needs a GPU).  The same gate set as the
// reference's device suite (tests/test_gpu.cu:54-1467), written against
// w4::gpu: bitwise dequant and hook output against the host dequant, GEMM and
// attention within rel L2 1e-3 of the FP64 host references, pairs of gated
// paths within 2e-3, dispatcher and paged outputs equal to their counterparts
// byte for byte.  The host headers used as references here are themselves
// checked byte for byte against the C oracle by test_host.
#include <cmath>
#include <cstring>
#include <numeric>
#include <random>
#include <vector>

#include "check.hpp"
#include "w4/dispatch.cuh"
#include "w4/kvflash.cuh"

using namespace w4;
using namespace w4::gpu;

namespace {

template <class T>
struct Dev {
  T* p = nullptr;
  size_t n = 0;
  Dev() = default;
  explicit Dev(size_t count) : n(count) {
    hip_check(hipMalloc((void**)&p, std::max<size_t>(count, 1) * sizeof(T)), "hipMalloc");
    hip_check(hipMemset(p, 0xEE, std::max<size_t>(count, 1) * sizeof(T)), "hipMemset");
  }
  explicit Dev(const std::vector<T>& host) : Dev(host.size()) {
    if (n) hip_check(hipMemcpy(p, host.data(), n * sizeof(T), hipMemcpyHostToDevice), "upload");
  }
  Dev(const Dev&) = delete;
  Dev& operator=(const Dev&) = delete;
  ~Dev() { (void)hipFree(p); }
  std::vector<T> get() const {
    hip_check(hipDeviceSynchronize(), "sync");
    std::vector<T> host(n);
    if (n) hip_check(hipMemcpy(host.data(), p, n * sizeof(T), hipMemcpyDeviceToHost), "download");
    return host;
  }
};

template <class T>
bool same(const std::vector<T>& a, const std::vector<T>& b) {
  return a.size() == b.size() && std::memcmp(a.data(), b.data(), a.size() * sizeof(T)) == 0;
}

// sqrt(sum (dev - ref)^2 / sum ref^2)
double rel_l2(const std::vector<__half>& dev, const std::vector<double>& ref) {
  double num = 0, den = 0;
  for (size_t i = 0; i < ref.size(); ++i) {
    const double d = (double)__half2float(dev[i]) - ref[i];
    num += d * d;
    den += ref[i] * ref[i];
  }
  return std::sqrt(num / (den > 0 ? den : 1.0));
}

double cross(const std::vector<__half>& a, const std::vector<__half>& b, const std::vector<double>& ref) {
  double num = 0, den = 0;
  for (size_t i = 0; i < ref.size(); ++i) {
    const double d = (double)__half2float(a[i]) - (double)__half2float(b[i]);
    num += d * d;
    den += ref[i] * ref[i];
  }
  return std::sqrt(num / (den > 0 ? den : 1.0));
}

double g_worst = 0;
void oracle_gate(Checks& t, const std::vector<__half>& dev, const std::vector<double>& ref, const char* what) {
  const double r = rel_l2(dev, ref);
  g_worst = std::max(g_worst, r);
  t.expect(r <= 1e-3, what);
}

struct Shape { int M, N, K, gs; };
const Shape kShapes[] = {{1, 64, 64, 8},    {8, 128, 96, 16},  {16, 256, 100, 32}, {4, 96, 72, 48},
                         {2, 32, 128, 64},  {3, 40, 256, 128}, {5, 72, 40, 8},     {17, 64, 128, 16},
                         {33, 48, 104, 24}, {20, 32, 100, 8},  {65, 96, 100, 16},  {1, 256, 4096, 128},
                         {12, 80, 2048, 32},
                         // long K: K-split vector kernel (M <= 2), pipelined matrix-core kernel above
                         {2, 32, 11008, 128}, {3, 32, 8192, 64},   {24, 16, 14336, 32}};

void gemm_gates(Checks& t) {
  const BlasHandle blas = make_blas();
  for (const bool sym : {true, false})
    for (size_t i = 0; i < sizeof kShapes / sizeof *kShapes; ++i) {
      const Shape c = kShapes[i];
      const uint64_t seed = 0x44A1ULL ^ (uint64_t)(i * 977 + (sym ? 0 : 1));
      const PackedW p = quantize(normal_weights(c.N * c.K, seed), c.N, c.K, c.gs, sym);
      const auto w_ref = dequant_all(p);
      const auto x = normal_activations(c.M * c.K, seed + 1);
      const auto ref = gemm_oracle(x, c.M, c.K, w_ref, c.N);
      Dev<uint32_t> q(p.q), z(p.zeros);
      Dev<__half> s(p.scales), xd(x), w((size_t)c.N * c.K), c2((size_t)c.M * c.N);
      const DevicePackedW dp{c.N, c.K, c.gs, p.G, sym ? 1 : 0, q.p, s.p, sym ? nullptr : z.p};
      dequant(dp, w.p);
      t.expect(same(w.get(), w_ref), "dequant bitwise");
      gemm_fp16(blas, w.p, xd.p, c2.p, c.M, c.N, c.K);
      const auto c_blas = c2.get();
      oracle_gate(t, c_blas, ref, "two-pass GEMM vs FP64 oracle");
      std::vector<__half> out[2];
      int which = 0;
      for (auto fn : {gemm_fused, gemm_mma}) {
        Dev<__half> cd((size_t)c.M * c.N), hook((size_t)c.N * c.K);
        fn(dp, xd.p, cd.p, c.M, 0, hook.p);
        t.expect(same(hook.get(), w_ref), "w_out bitwise");
        out[which] = cd.get();
        oracle_gate(t, out[which], ref, "fused GEMM vs FP64 oracle");
        t.expect(cross(out[which], c_blas, ref) <= 2e-3, "fused GEMM vs two-pass");
        ++which;
      }
      Dev<__half> cd((size_t)c.M * c.N), hook((size_t)c.N * c.K);
      gemm(dp, xd.p, cd.p, c.M, 0, hook.p);
      t.expect(same(hook.get(), w_ref), "dispatcher w_out bitwise");
      t.expect(same(cd.get(), out[c.M < dispatch_mma_min_m(c.N, c.K) ? 0 : 1]), "dispatcher output == its callee");
    }
  for (size_t i = 0; i < sizeof kShapes / sizeof *kShapes; ++i) {
    const Shape c = kShapes[i];
    const uint64_t seed = 0x1E4AULL ^ (uint64_t)(i * 977);
    const mx::PackedWm p = mx::quantize_mx(normal_weights(c.N * c.K, seed), c.N, c.K);
    const auto w_ref = mx::dequant_all_mx(p);
    const auto x = normal_activations(c.M * c.K, seed + 1);
    const auto ref = gemm_oracle(x, c.M, c.K, w_ref, c.N);
    Dev<uint32_t> q(p.q);
    Dev<uint8_t> s(p.scales);
    Dev<__half> xd(x), w((size_t)c.N * c.K);
    const DevicePackedWm dp{c.N, c.K, p.B, q.p, s.p};
    dequant_mx(dp, w.p);
    t.expect(same(w.get(), w_ref), "mx dequant bitwise");
    std::vector<__half> out[2];
    int which = 0;
    for (auto fn : {gemm_fused_mx, gemm_mma_mx}) {
      Dev<__half> cd((size_t)c.M * c.N), hook((size_t)c.N * c.K);
      fn(dp, xd.p, cd.p, c.M, 0, hook.p);
      t.expect(same(hook.get(), w_ref), "mx w_out bitwise");
      out[which] = cd.get();
      oracle_gate(t, out[which], ref, "mx GEMM vs FP64 oracle");
      ++which;
    }
    t.expect(cross(out[0], out[1], ref) <= 2e-3, "mx vector vs matrix kernel");
    Dev<__half> cd((size_t)c.M * c.N);
    gemm_mx(dp, xd.p, cd.p, c.M);
    t.expect(same(cd.get(), out[c.M < dispatch_mma_min_m_mx(c.N, c.K) ? 0 : 1]), "mx dispatcher output == its callee");
  }
}

struct KvDev {
  Dev<uint32_t> qk, qv, zk, zv;
  Dev<__half> sk, sv;
  DeviceKVW4 view;
  explicit KvDev(const kv::KVCacheW4& c)
      : qk(c.q_k), qv(c.q_v), zk(c.z_k), zv(c.z_v), sk(c.s_k), sv(c.s_v),
        view{c.H, c.S, c.D, c.gs, c.G, c.symmetric ? 1 : 0, qk.p, sk.p, c.symmetric ? nullptr : zk.p,
             qv.p, sv.p, c.symmetric ? nullptr : zv.p} {}
};

std::vector<__half> all_heads(const kv::KVCacheW4& c, bool vside) {
  std::vector<__half> out;
  for (int h = 0; h < c.H; ++h) {
    const auto slab = kv::dequant_head(c, h, vside);
    out.insert(out.end(), slab.begin(), slab.end());
  }
  return out;
}

// runs the W4 flash gates for one cache and returns the output bytes
std::vector<__half> w4_flash_gates(Checks& t, const kv::KVCacheW4& c, const std::vector<__half>& q) {
  const auto ref = kv::attention_reference(q, c);
  const auto kd = all_heads(c, false), vd = all_heads(c, true);
  KvDev d(c);
  Dev<__half> qd(q), out((size_t)c.H * c.D), ko(kd.size()), vo(vd.size());
  attention_w4_flash(d.view, qd.p, out.p, 0, ko.p, vo.p);
  t.expect(same(ko.get(), kd) && same(vo.get(), vd), "flash k_out / v_out bitwise");
  const auto o = out.get();
  oracle_gate(t, o, ref, "W4 flash vs FP64 reference");
  Dev<__half> k16(kd), v16(vd), o16((size_t)c.H * c.D);
  attention_fp16_flash(qd.p, k16.p, v16.p, o16.p, c.H, c.S, c.D);
  const auto of = o16.get();
  oracle_gate(t, of, ref, "FP16 flash vs FP64 reference");
  t.expect(cross(o, of, ref) <= 2e-3, "W4 flash vs FP16 flash");
  if (c.S <= KV_MAX_S) {  // the single-pass entry points (kvattention.cuh:226-249) accept this length
    Dev<__half> o1((size_t)c.H * c.D), o2((size_t)c.H * c.D);
    attention_w4(d.view, qd.p, o1.p);
    attention_fp16(qd.p, k16.p, v16.p, o2.p, c.H, c.S, c.D);
    oracle_gate(t, o1.get(), ref, "W4 single-pass entry vs FP64 reference");
    t.expect(cross(o1.get(), o2.get(), ref) <= 2e-3, "W4 vs FP16 single-pass entries");
  }
  return o;
}

void attention_gates(Checks& t) {
  struct A { int H, S, D, gs; };
  const A cfgs[] = {{1, 1, 64, 32}, {2, 7, 64, 8}, {4, 128, 128, 128}, {2, 300, 96, 32}, {3, 65, 40, 8},
                    {1, 4096, 64, 64}, {2, 5000, 64, 32}, {1, 9000, 128, 64}};
  for (const bool sym : {true, false})
    for (size_t i = 0; i < sizeof cfgs / sizeof *cfgs; ++i) {
      const A a = cfgs[i];
      const uint64_t seed = 0x77B5ULL ^ (uint64_t)(i * 977 + (sym ? 0 : 1));
      const auto c = kv::quantize_cache(normal_weights(a.H * a.S * a.D, seed),
                                        normal_weights(a.H * a.S * a.D, seed + 1), a.H, a.S, a.D, a.gs, sym);
      w4_flash_gates(t, c, normal_activations(a.H * a.D, seed + 2));
    }
  // FP8
  const A f8[] = {{1, 1, 64, 32}, {2, 7, 64, 8}, {4, 128, 128, 128}, {2, 300, 96, 32}, {3, 65, 40, 8},
                  {1, 9000, 128, 64}};
  for (size_t i = 0; i < sizeof f8 / sizeof *f8; ++i) {
    const A a = f8[i];
    const uint64_t seed = 0xF80AULL ^ (uint64_t)(i * 977);
    const auto c = kv8::quantize_cache_f8(normal_weights(a.H * a.S * a.D, seed),
                                          normal_weights(a.H * a.S * a.D, seed + 1), a.H, a.S, a.D, a.gs);
    const auto q = normal_activations(a.H * a.D, seed + 2);
    const auto ref = kv8::attention_reference_f8(q, c);
    std::vector<__half> kd, vd;
    for (int h = 0; h < a.H; ++h) {
      const auto ks = kv8::dequant_head_f8(c, h, false), vs = kv8::dequant_head_f8(c, h, true);
      kd.insert(kd.end(), ks.begin(), ks.end());
      vd.insert(vd.end(), vs.begin(), vs.end());
    }
    Dev<uint8_t> qk(c.q_k), qv(c.q_v);
    Dev<__half> sk(c.s_k), sv(c.s_v), qd(q), out((size_t)a.H * a.D), ko(kd.size()), vo(vd.size());
    const DeviceKVF8 view{a.H, a.S, a.D, a.gs, c.G, qk.p, sk.p, qv.p, sv.p};
    attention_f8_flash(view, qd.p, out.p, 0, ko.p, vo.p);
    t.expect(same(ko.get(), kd) && same(vo.get(), vd), "f8 flash hooks bitwise");
    oracle_gate(t, out.get(), ref, "FP8 flash vs FP64 reference");
    Dev<__half> k16(kd.size());
    dequant_f8(qk.p, sk.p, k16.p, a.H * a.S, a.D, a.gs);
    t.expect(same(k16.get(), kd), "dequant_f8 bitwise");
  }
  // paged: output and hooks equal the contiguous kernel byte for byte
  struct P { int H, S, D, gs, page; };
  const P paged[] = {{2, 300, 96, 32, 16}, {2, 520, 64, 32, 16}, {1, 1000, 128, 64, 64}, {3, 65, 40, 8, 32},
                     {1, 5000, 64, 32, 256}};
  for (const bool sym : {true, false})
    for (size_t i = 0; i < sizeof paged / sizeof *paged; ++i) {
      const P a = paged[i];
      const uint64_t seed = 0x9A6EULL ^ (uint64_t)(i * 977 + (sym ? 0 : 1));
      const auto c = kv::quantize_cache(normal_weights(a.H * a.S * a.D, seed),
                                        normal_weights(a.H * a.S * a.D, seed + 1), a.H, a.S, a.D, a.gs, sym);
      const auto q = normal_activations(a.H * a.D, seed + 2);
      const auto contiguous = w4_flash_gates(t, c, q);
      std::vector<int> bt((size_t)(a.S + a.page - 1) / a.page);
      std::iota(bt.begin(), bt.end(), 0);
      std::mt19937_64 rng(seed ^ 0x5ED);
      std::shuffle(bt.begin(), bt.end(), rng);
      const auto pc = kv::paged_from_contiguous(c, a.page, bt);
      kv::validate_paged(pc);
      Dev<uint32_t> qk(pc.q_k), qv(pc.q_v), zk(pc.z_k), zv(pc.z_v);
      Dev<__half> sk(pc.s_k), sv(pc.s_v), qd(q), out((size_t)a.H * a.D);
      Dev<__half> ko((size_t)a.H * a.S * a.D), vo((size_t)a.H * a.S * a.D);
      Dev<int> btd(bt);
      const DeviceKVW4 view{a.H, a.S, a.D, a.gs, c.G, sym ? 1 : 0, qk.p, sk.p, sym ? nullptr : zk.p,
                            qv.p, sv.p, sym ? nullptr : zv.p};
      attention_w4_flash_paged(view, btd.p, a.page, pc.npages, qd.p, out.p, 0, ko.p, vo.p);
      t.expect(same(out.get(), contiguous), "paged output == contiguous output");
      t.expect(same(ko.get(), all_heads(c, false)) && same(vo.get(), all_heads(c, true)), "paged hooks bitwise");
    }
  // grouped queries: equal to the plain call on a cache with each slab repeated
  {
    const int H = 2, S = 777, D = 128, gs = 32, group = 4;
    const auto c = kv::quantize_cache(normal_weights(H * S * D, 0x61), normal_weights(H * S * D, 0x62), H, S, D,
                                      gs, true);
    const auto q = normal_activations(H * group * D, 0x63);
    const auto ref = kv::attention_reference_gqa(q, c, group);
    KvDev d(c);
    Dev<__half> qd(q), out((size_t)H * group * D);
    attention_w4_flash_gqa(d.view, group, qd.p, out.p);
    oracle_gate(t, out.get(), ref, "grouped-query W4 flash vs FP64 reference");
  }
}

// The device quantizers against the host ones of the same headers
// (pack.hpp:64-130, mx.hpp:71-119, kvcache.hpp:60-108, kvfp8.hpp:70-128): same
// bytes, same exceptions.
template <class F>
bool throws_invalid(F&& f, const char* text) {
  try {
    f();
  } catch (const std::invalid_argument& e) {
    return std::strstr(e.what(), text) != nullptr;
  } catch (...) {
  }
  return false;
}

void quantizer_gates(Checks& t) {
  Dev<int> status(1);
  const Shape shapes[] = {{0, 5, 200, 64}, {0, 3, 1001, 128}, {0, 7, 100, 24}, {0, 64, 4096, 128}};
  for (const Shape& c : shapes)
    for (const bool sym : {true, false}) {
      auto w = normal_weights(c.N * c.K, 0x51u + (unsigned)c.K);
      for (size_t i = 0; i < w.size(); i += 3) w[i] *= 9.0;  // heavier tails
      const PackedW ref = quantize(w, c.N, c.K, c.gs, sym);
      Dev<double> wd(w);
      Dev<uint32_t> q(ref.q.size()), z(ref.zeros.size());
      Dev<__half> s(ref.scales.size());
      const DevicePackedW out{c.N, c.K, c.gs, ref.G, sym ? 1 : 0, q.p, s.p, sym ? nullptr : z.p};
      gpu::quantize(out, wd.p, status.p);
      t.expect(same(q.get(), ref.q) && same(s.get(), ref.scales), "device quantize: codes, scales");
      if (!sym) t.expect(same(z.get(), ref.zeros), "device quantize: zero-points");
    }
  {
    const int N = 6, K = 1000;
    auto w = normal_weights(N * K, 77);
    const mx::PackedWm ref = mx::quantize_mx(w, N, K);
    Dev<double> wd(w);
    Dev<uint32_t> q(ref.q.size());
    Dev<uint8_t> s(ref.scales.size());
    const DevicePackedWm out{N, K, ref.B, q.p, s.p};
    gpu::quantize_mx(out, wd.p, status.p);
    t.expect(same(q.get(), ref.q) && same(s.get(), ref.scales), "device quantize_mx");
    w[123] = std::nan("");
    Dev<double> bad(w);
    t.expect(throws_invalid([&] { gpu::quantize_mx(out, bad.p, status.p); },
                            "quantize_mx: non-finite input"),
             "device quantize_mx throws on NaN");
  }
  {
    const int H = 3, S = 65, D = 128, gs = 32;
    const auto k = normal_weights(H * S * D, 5), v = normal_weights(H * S * D, 6);
    Dev<double> kd(k), vd(v);
    for (const bool sym : {true, false}) {
      const kv::KVCacheW4 ref = kv::quantize_cache(k, v, H, S, D, gs, sym);
      Dev<uint32_t> qk(ref.q_k.size()), qv(ref.q_v.size()), zk(ref.z_k.size()), zv(ref.z_v.size());
      Dev<__half> sk(ref.s_k.size()), sv(ref.s_v.size());
      const DeviceKVW4 out{H, S, D, gs, ref.G, sym ? 1 : 0, qk.p, sk.p, sym ? nullptr : zk.p,
                           qv.p, sv.p, sym ? nullptr : zv.p};
      gpu::quantize_cache(out, kd.p, vd.p, status.p);
      t.expect(same(qk.get(), ref.q_k) && same(qv.get(), ref.q_v) && same(sk.get(), ref.s_k) &&
                   same(sv.get(), ref.s_v),
               "device quantize_cache: codes, scales");
      if (!sym)
        t.expect(same(zk.get(), ref.z_k) && same(zv.get(), ref.z_v),
                 "device quantize_cache: zero-points");
    }
    const kv8::KVCacheF8 ref8 = kv8::quantize_cache_f8(k, v, H, S, D, gs);
    Dev<uint8_t> qk(ref8.q_k.size()), qv(ref8.q_v.size());
    Dev<__half> sk(ref8.s_k.size()), sv(ref8.s_v.size());
    const DeviceKVF8 out8{H, S, D, gs, ref8.G, qk.p, sk.p, qv.p, sv.p};
    gpu::quantize_cache_f8(out8, kd.p, vd.p, status.p);
    t.expect(same(qk.get(), ref8.q_k) && same(qv.get(), ref8.q_v) && same(sk.get(), ref8.s_k) &&
                 same(sv.get(), ref8.s_v),
             "device quantize_cache_f8");
    auto big = v;
    big[7] = 1e9;
    Dev<double> bigd(big);
    t.expect(throws_invalid([&] { gpu::quantize_cache_f8(out8, kd.p, bigd.p, status.p); },
                            "group scale outside FP16 range"),
             "device quantize_cache_f8 throws on a scale beyond FP16");
  }
}

// W4A4: activations quantized on the device equal the host quantizer's bytes, and
// the product of the two packed operands is within 1e-3 of the FP64 product of
// their dequantized values (mx.hpp:131-140, pack.hpp:150-170).
void w4a4_gates(Checks& t) {
  Dev<int> status(1);
  const Shape shapes[] = {{5, 100, 1000, 0}, {64, 128, 1024, 0}, {400, 300, 512, 0}};
  for (const Shape& c : shapes) {
    const mx::PackedWm w = mx::quantize_mx(normal_weights(c.N * c.K, 31), c.N, c.K);
    const auto x16 = normal_activations(c.M * c.K, 32);
    std::vector<double> xd(x16.size());
    for (size_t i = 0; i < xd.size(); ++i) xd[i] = (double)__half2float(x16[i]);
    const mx::PackedWm xq = mx::quantize_mx(xd, c.M, c.K);
    const auto ref = gemm_oracle(mx::dequant_all_mx(xq), c.M, c.K, mx::dequant_all_mx(w), c.N);
    Dev<uint32_t> wq(w.q), xqd(xq.q.size());
    Dev<uint8_t> wsc(w.scales), xsd(xq.scales.size());
    Dev<__half> x(x16), out((size_t)c.M * c.N);
    const DevicePackedWm dw{c.N, c.K, w.B, wq.p, wsc.p}, dx{c.M, c.K, xq.B, xqd.p, xsd.p};
    quantize_mx_f16_async(dx, x.p, status.p);
    t.expect(same(xqd.get(), xq.q) && same(xsd.get(), xq.scales) && status.get()[0] == 0,
             "activations quantized on the device: host bytes");
    gemm_mx_w4a4(dw, dx, out.p);
    oracle_gate(t, out.get(), ref, "W4A4 product vs FP64 product of the dequantized operands");
  }
}

// W4A8: the same gates with MXFP8 activations (include/w4/mxact.hpp).
void w4a8_gates(Checks& t) {
  Dev<int> status(1);
  const Shape shapes[] = {{5, 100, 992, 0}, {64, 128, 1024, 0}, {200, 72, 512, 0}};
  for (const Shape& c : shapes) {
    const mx::PackedWm w = mx::quantize_mx(normal_weights(c.N * c.K, 41), c.N, c.K);
    const auto x16 = normal_activations(c.M * c.K, 42);
    std::vector<double> xd(x16.size());
    for (size_t i = 0; i < xd.size(); ++i) xd[i] = (double)__half2float(x16[i]);
    const mxa::PackedXm8 xq = mxa::quantize_mx8(xd, c.M, c.K);
    const auto ref = mxa::gemm_reference_w4a8(xq, w);
    Dev<uint32_t> wq(w.q);
    Dev<uint8_t> wsc(w.scales), xqd(xq.q.size()), xsd(xq.scales.size());
    Dev<__half> x(x16), out((size_t)c.M * c.N);
    const DevicePackedWm dw{c.N, c.K, w.B, wq.p, wsc.p};
    const DeviceActMx8 dx{c.M, c.K, xq.B, xqd.p, xsd.p};
    quantize_mx8_f16_async(dx, x.p, status.p);
    t.expect(same(xqd.get(), xq.q) && same(xsd.get(), xq.scales) && status.get()[0] == 0,
             "MXFP8 activations quantized on the device: host bytes");
    gemm_mx_w4a8(dw, dx, out.p);
    oracle_gate(t, out.get(), ref, "W4A8 product vs FP64 product of the dequantized operands");
  }
}

}  // namespace

int main() {
  int ndev = 0;
  if (hipGetDeviceCount(&ndev) != hipSuccess || ndev < 1) {
    std::printf("device: no GPU visible\n");
    return 77;
  }
  Checks t;
  gemm_gates(t);
  attention_gates(t);
  quantizer_gates(t);
  w4a4_gates(t);
  w4a8_gates(t);
  std::printf("worst rel L2 vs the FP64 references = %.3e\n", g_worst);
  return t.finish("device");
}
