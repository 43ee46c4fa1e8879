// Entry contracts of the w4::gpu API, runnable without a GPU: every malformed
// call must throw std::invalid_argument before anything is dereferenced,
// allocated or launched, so all device pointers here are the dummy address 1.
// The cases are the ones the reference device suite pins
// (tests/test_gpu.cu:1471-1864), minus the two single-block attention kernels.
#include <climits>

#include "check.hpp"
#include "w4/dispatch.cuh"
#include "w4/kvflash.cuh"

using namespace w4::gpu;

int main() {
  Checks t;
  __half* const P = (__half*)1;
  const uint32_t* const U = (const uint32_t*)1;
  const DevicePackedW ok{2, 32, 8, 4, 1, U, P, nullptr};

  // -- structural faults shared by dequant / fused / mma / dispatcher
  struct Fault { const char* name; DevicePackedW view; };
  auto with = [&](auto edit) { DevicePackedW v = ok; edit(v); return v; };
  const Fault faults[] = {
      {"N=0", with([](auto& v) { v.N = 0; })},
      {"K=0", with([](auto& v) { v.K = 0; })},
      {"gs=0", with([](auto& v) { v.gs = 0; })},
      {"gs=7", with([](auto& v) { v.gs = 7; })},
      {"G wrong", with([](auto& v) { v.G = 3; })},
      {"q null", with([](auto& v) { v.q = nullptr; })},
      {"scales null", with([](auto& v) { v.scales = nullptr; })},
      {"asym without zeros", with([](auto& v) { v.symmetric = 0; })},
      {"sym with zeros", with([&](auto& v) { v.zeros = U; })},
  };
  for (const auto& f : faults) {
    t.throws_invalid([&] { dequant(f.view, P); }, f.name);
    t.throws_invalid([&] { gemm_fused(f.view, P, P, 2); }, f.name);
    t.throws_invalid([&] { gemm_mma(f.view, P, P, 2); }, f.name);
    t.throws_invalid([&] { gemm(f.view, P, P, 1); }, f.name);
    t.throws_invalid([&] { gemm(f.view, P, P, 16); }, f.name);
  }
  t.throws_invalid([&] { dequant(ok, nullptr); }, "dequant w null");
  // 2^21 rows x 1024 words reaches 2^31 exactly
  t.throws_invalid([&] { dequant(with([](auto& v) { v.N = 1 << 21; v.K = 8192; v.G = 1024; }), P); },
                   "dequant N*words(K) = 2^31");
  for (auto fn : {gemm_fused, gemm_mma, gemm}) {
    t.throws_invalid([&] { fn(ok, nullptr, P, 2, 0, nullptr); }, "x null");
    t.throws_invalid([&] { fn(ok, P, nullptr, 2, 0, nullptr); }, "c null");
    t.throws_invalid([&] { fn(ok, P, P, 0, 0, nullptr); }, "M=0");
    t.throws_invalid([&] { fn(ok, P, P, -3, 0, nullptr); }, "M<0");
  }
  t.throws_invalid([&] { gemm_fused(ok, P, P, 262141); }, "fused M past its grid bound");
  t.throws_invalid([&] { gemm_mma(ok, P, P, 4194241); }, "mma M past its grid bound");
  t.throws_invalid([&] { gemm(ok, P, P, 4194241); }, "dispatcher inherits the mma bound");
  t.throws_invalid([&] { gemm_mma(with([](auto& v) { v.N = INT_MAX; }), P, P, 2); }, "mma N overflow");
  t.throws_invalid([&] { gemm_fused(with([](auto& v) { v.N = INT_MAX; }), P, P, 2); }, "fused N overflow");
  t.throws_invalid([&] { gemm_fp16(make_blas(), P, P, P, 0, 2, 2); }, "gemm_fp16 M=0");
  t.throws_invalid([&] { gemm_fp16(make_blas(), nullptr, P, P, 2, 2, 2); }, "gemm_fp16 w null");

  // -- MXFP4
  const DevicePackedWm okm{2, 32, 1, U, (const uint8_t*)1};
  auto withm = [&](auto edit) { DevicePackedWm v = okm; edit(v); return v; };
  const DevicePackedWm mfaults[] = {withm([](auto& v) { v.N = 0; }), withm([](auto& v) { v.B = 2; }),
                                    withm([](auto& v) { v.q = nullptr; }),
                                    withm([](auto& v) { v.scales = nullptr; })};
  for (const auto& v : mfaults) {
    t.throws_invalid([&] { dequant_mx(v, P); }, "mx dequant view");
    t.throws_invalid([&] { gemm_fused_mx(v, P, P, 2); }, "mx fused view");
    t.throws_invalid([&] { gemm_mma_mx(v, P, P, 2); }, "mx mma view");
    t.throws_invalid([&] { gemm_mx(v, P, P, 2); }, "mx dispatch view, vector side");
    t.throws_invalid([&] { gemm_mx(v, P, P, 16); }, "mx dispatch view, matrix side");
    t.throws_invalid([&] { validate_mx(v); }, "validate_mx");
  }
  t.throws_invalid([&] { dequant_mx(okm, nullptr); }, "mx dequant w null");
  t.throws_invalid([&] { dequant_mx(withm([](auto& v) { v.N = 1 << 21; v.K = 8192; v.B = 256; }), P); },
                   "mx dequant N*words(K) = 2^31");
  for (auto fn : {gemm_fused_mx, gemm_mma_mx, gemm_mx}) {
    t.throws_invalid([&] { fn(okm, nullptr, P, 2, 0, nullptr); }, "mx x null");
    t.throws_invalid([&] { fn(okm, P, nullptr, 2, 0, nullptr); }, "mx c null");
    t.throws_invalid([&] { fn(okm, P, P, 0, 0, nullptr); }, "mx M=0");
  }
  t.throws_invalid([&] { gemm_fused_mx(okm, P, P, 262141); }, "mx fused M bound");
  t.throws_invalid([&] { gemm_mma_mx(okm, P, P, 4194241); }, "mx mma M bound");
  t.throws_invalid([&] { gemm_mx(okm, P, P, 4194241); }, "mx dispatcher M bound");
  t.throws_invalid([&] { gemm_fused_mx(withm([](auto& v) { v.N = INT_MAX; }), P, P, 2); }, "mx fused N overflow");
  t.throws_invalid([&] { gemm_mma_mx(withm([](auto& v) { v.N = INT_MAX; }), P, P, 2); }, "mx mma N overflow");

  // -- W4 flash attention (contiguous, grouped, paged)
  const DeviceKVW4 okv{1, 4, 8, 8, 1, 1, U, P, nullptr, U, P, nullptr};
  auto withk = [&](auto edit) { DeviceKVW4 v = okv; edit(v); return v; };
  const DeviceKVW4 kfaults[] = {
      withk([](auto& v) { v.H = 0; }), withk([](auto& v) { v.S = 0; }), withk([](auto& v) { v.D = 0; }),
      withk([](auto& v) { v.D = 513; v.G = 65; }), withk([](auto& v) { v.gs = 7; }),
      withk([](auto& v) { v.gs = 0; }), withk([](auto& v) { v.G = 2; }),
      withk([](auto& v) { v.q_k = nullptr; }), withk([](auto& v) { v.s_v = nullptr; }),
      withk([](auto& v) { v.symmetric = 0; }), withk([&](auto& v) { v.z_k = U; }),
      withk([](auto& v) { v.S = 65535 * 256 + 1; })};
  const int* BT = (const int*)1;
  for (const auto& v : kfaults) {
    t.throws_invalid([&] { attention_w4_flash(v, P, P); }, "kv flash view");
    t.throws_invalid([&] { attention_w4_flash_gqa(v, 4, P, P); }, "kv flash gqa view");
    t.throws_invalid([&] { attention_w4_flash_paged(v, BT, 16, 1 << 20, P, P); }, "kv paged view");
  }
  t.throws_invalid([&] { attention_w4(withk([](auto& v) { v.S = KV_MAX_S + 1; }), P, P); }, "kv single-pass S bound");
  t.throws_invalid([&] { attention_w4(okv, nullptr, P); }, "kv single-pass q null");
  t.throws_invalid([&] { attention_fp16(P, P, P, P, 1, KV_MAX_S + 1, 64); }, "kv fp16 single-pass S bound");
  t.throws_invalid([&] { attention_fp16(P, P, nullptr, P, 1, 64, 64); }, "kv fp16 single-pass null");
  t.throws_invalid([&] { attention_w4_flash(okv, nullptr, P); }, "kv flash q null");
  t.throws_invalid([&] { attention_w4_flash(okv, P, nullptr); }, "kv flash out null");
  t.throws_invalid([&] { attention_w4_flash_gqa(okv, 0, P, P); }, "kv flash group=0");
  t.throws_invalid([&] { attention_w4_flash_paged(okv, nullptr, 16, 1, P, P); }, "paged bt null");
  t.throws_invalid([&] { attention_w4_flash_paged(okv, BT, 0, 1, P, P); }, "paged page=0");
  t.throws_invalid([&] { attention_w4_flash_paged(okv, BT, 16, 0, P, P); }, "paged npages=0");
  t.throws_invalid([&] { attention_w4_flash_paged(withk([](auto& v) { v.S = 100; }), BT, 16, 1, P, P); },
                   "paged pool smaller than S");
  t.throws_invalid([&] { attention_w4_flash_paged(okv, BT, 50000, 50000, P, P); }, "paged pool rows >= 2^31");
  t.throws_invalid([&] { attention_w4_flash_paged(okv, BT, 16, 1, nullptr, P); }, "paged q null");
  t.throws_invalid([&] { attention_w4_flash_paged_batched(okv, BT, 0, 1, 16, 1, 1, P, P); }, "paged batch nseq=0");
  t.throws_invalid([&] { attention_w4_flash_paged_batched(okv, BT, 2, 0, 16, 1, 1, P, P); }, "paged batch stride");

  // -- FP16 flash
  t.throws_invalid([&] { attention_fp16_flash(P, P, P, P, 0, 4, 8); }, "fp16 flash H=0");
  t.throws_invalid([&] { attention_fp16_flash(P, P, P, P, 1, 4, 513); }, "fp16 flash D bound");
  t.throws_invalid([&] { attention_fp16_flash(P, P, P, P, 1, 65535 * 256 + 1, 8); }, "fp16 flash S bound");
  t.throws_invalid([&] { attention_fp16_flash(nullptr, P, P, P, 1, 4, 8); }, "fp16 flash q null");
  t.throws_invalid([&] { attention_fp16_flash(P, P, nullptr, P, 1, 4, 8); }, "fp16 flash v null");

  // -- FP8 flash and dequant_f8 (byte caches must be 4-byte aligned: address 4 is, 1 is not)
  const uint8_t* const B4 = (const uint8_t*)4;
  const DeviceKVF8 ok8{1, 4, 8, 8, 1, B4, P, B4, P};
  auto with8 = [&](auto edit) { DeviceKVF8 v = ok8; edit(v); return v; };
  const DeviceKVF8 f8faults[] = {
      with8([](auto& v) { v.S = 0; }), with8([](auto& v) { v.D = 513; v.G = 65; }),
      with8([](auto& v) { v.D = 2; v.G = 1; }), with8([](auto& v) { v.gs = 7; }),
      with8([](auto& v) { v.G = 3; }), with8([](auto& v) { v.q_k = nullptr; }),
      with8([](auto& v) { v.S = 65535 * 256 + 1; }),
      with8([](auto& v) { v.q_k = (const uint8_t*)1; }), with8([](auto& v) { v.q_v = (const uint8_t*)6; })};
  for (const auto& v : f8faults) {
    t.throws_invalid([&] { attention_f8_flash(v, P, P); }, "f8 flash view");
    t.throws_invalid([&] { attention_f8_flash_gqa(v, 2, 1, P, P); }, "f8 flash gqa view");
  }
  t.throws_invalid([&] { attention_f8_flash(ok8, nullptr, P); }, "f8 flash q null");
  t.throws_invalid([&] { attention_f8_flash_gqa(ok8, 1, 2, P, P); }, "f8 flash scale mode");
  t.throws_invalid([&] { dequant_f8(nullptr, P, P, 4, 8, 8); }, "f8 dequant q null");
  t.throws_invalid([&] { dequant_f8(B4, P, P, 4, 6, 8); }, "f8 dequant D%4");
  t.throws_invalid([&] { dequant_f8(B4, P, P, 4, 8, 7); }, "f8 dequant gs=7");
  t.throws_invalid([&] { dequant_f8((const uint8_t*)3, P, P, 4, 8, 8); }, "f8 dequant misaligned");
  t.throws_invalid([&] { dequant_f8(B4, P, P, 0, 8, 8); }, "f8 dequant S=0");
  t.throws_invalid([&] { dequant_f8(B4, P, P, 1 << 30, 8, 8); }, "f8 dequant 2^31 words");
  return t.finish("contracts");
}
