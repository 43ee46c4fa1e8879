#pragma once

// w4::gpu -- the device entry points of the fused-dequant path, as thin C++
// wrappers over the C ABI of libw4amd.so (include/w4_abi.h).  Signatures follow
// the reference's launch wrappers (dequant.cuh, fused.cuh, mma.cuh,
// mxfused.cuh, dispatch.cuh, kvattention.cuh, kvflash.cuh; cited per function)
// with hipStream_t in place of cudaStream_t.  Contract violations throw
// std::invalid_argument before anything touches the device; HIP failures throw
// std::runtime_error.  All pointers are device pointers owned by the caller;
// launches are asynchronous on `stream`.
//
// Link with -lw4amd.

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <cstdint>
#include <stdexcept>
#include <string>

#include "../w4_abi.h"
#include "kvcache.hpp"
#include "kvfp8.hpp"
#include "kvpaged.hpp"
#include "mx.hpp"
#include "mxact.hpp"
#include "pack.hpp"

namespace w4::gpu {

// dequant.cuh:19-23
inline void hip_check(hipError_t e, const char* what) {
  if (e != hipSuccess) throw std::runtime_error(std::string(what) + ": " + hipGetErrorString(e));
}

// dequant.cuh:31-37 (field order and types are the ABI's)
struct DevicePackedW {
  int N, K, gs, G;
  int symmetric;
  const uint32_t* q;
  const __half* scales;
  const uint32_t* zeros;
};

// mxfused.cuh:26-30
struct DevicePackedWm {
  int N, K, B;
  const uint32_t* q;
  const uint8_t* scales;
};

// kvattention.cuh:39-48
struct DeviceKVW4 {
  int H, S, D, gs, G;
  int symmetric;
  const uint32_t* q_k;
  const __half* s_k;
  const uint32_t* z_k;
  const uint32_t* q_v;
  const __half* s_v;
  const uint32_t* z_v;
};

// kvflash.cuh:390-396
struct DeviceKVF8 {
  int H, S, D, gs, G;
  const uint8_t* q_k;
  const __half* s_k;
  const uint8_t* q_v;
  const __half* s_v;
};

constexpr int KV_MAX_S = 4096;   // kvattention.cuh:36
constexpr int KV_MAX_D = 512;    // kvattention.cuh:37
constexpr int FLASH_TILE = 256;  // kvflash.cuh:35

namespace detail {

inline void raise(int rc) {
  if (rc == W4_OK) return;
  const std::string msg = w4_last_error();
  if (rc == W4_EINVAL) throw std::invalid_argument(msg);
  throw std::runtime_error(msg);
}

inline const w4_half* h(const __half* p) { return reinterpret_cast<const w4_half*>(p); }
inline w4_half* h(__half* p) { return reinterpret_cast<w4_half*>(p); }

inline w4_packed_view abi(const DevicePackedW& p) {
  return w4_packed_view{p.N, p.K, p.gs, p.G, p.symmetric, p.q, h(p.scales), p.zeros};
}
inline w4_packed_mx_view abi(const DevicePackedWm& p) {
  return w4_packed_mx_view{p.N, p.K, p.B, p.q, p.scales};
}
inline w4_kv_view abi(const DeviceKVW4& p) {
  return w4_kv_view{p.H, p.S, p.D, p.gs, p.G, p.symmetric, p.q_k, h(p.s_k), p.z_k,
                    p.q_v, h(p.s_v), p.z_v};
}
inline w4_kv_f8_view abi(const DeviceKVF8& p) {
  return w4_kv_f8_view{p.H, p.S, p.D, p.gs, p.G, p.q_k, h(p.s_k), p.q_v, h(p.s_v)};
}

}  // namespace detail

// dispatch.cuh:25 -- the activation-row count from which gemm()/gemm_mx() use
// the matrix-core kernel, as measured on MI355X.
inline int dispatch_mma_min_m() { return w4_dispatch_mma_min_m(); }
inline int dispatch_mma_min_m(int N, int K) { return w4_dispatch_mma_min_m_for(N, K); }
inline int dispatch_mma_min_m(int N, int K, int gs) { return w4_dispatch_mma_min_m_for_gs(N, K, gs); }
inline int dispatch_mma_min_m_mx(int N, int K) { return w4_dispatch_mma_min_m_for_mx(N, K); }

// dequant.cuh:62-82
inline void dequant(const DevicePackedW& p, __half* w, hipStream_t stream = 0) {
  const auto v = detail::abi(p);
  detail::raise(w4_dequant(&v, detail::h(w), stream));
}

// fused.cuh:172-214
inline void gemm_fused(const DevicePackedW& p, const __half* x, __half* c, int M,
                       hipStream_t stream = 0, __half* w_out = nullptr) {
  const auto v = detail::abi(p);
  detail::raise(w4_gemm_fused(&v, detail::h(x), detail::h(c), M, stream, detail::h(w_out)));
}

// mma.cuh:234-260
inline void gemm_mma(const DevicePackedW& p, const __half* x, __half* c, int M,
                     hipStream_t stream = 0, __half* w_out = nullptr) {
  const auto v = detail::abi(p);
  detail::raise(w4_gemm_mma(&v, detail::h(x), detail::h(c), M, stream, detail::h(w_out)));
}

// dispatch.cuh:27-34
inline void gemm(const DevicePackedW& p, const __half* x, __half* c, int M,
                 hipStream_t stream = 0, __half* w_out = nullptr) {
  const auto v = detail::abi(p);
  detail::raise(w4_gemm(&v, detail::h(x), detail::h(c), M, stream, detail::h(w_out)));
}

// mxfused.cuh:32-37
inline void validate_mx(const DevicePackedWm& p) {
  w4::detail::require(p.N >= 1 && p.K >= 1, "mx: bad dims");
  w4::detail::require(p.B == mx::blocks(p.K), "mx: B inconsistent with K");
  w4::detail::require(p.q && p.scales, "mx: null pointer");
}

// mxfused.cuh:57-69
inline void dequant_mx(const DevicePackedWm& p, __half* w, hipStream_t stream = 0) {
  const auto v = detail::abi(p);
  detail::raise(w4_dequant_mx(&v, detail::h(w), stream));
}

// mxfused.cuh:166-198
inline void gemm_fused_mx(const DevicePackedWm& p, const __half* x, __half* c, int M,
                          hipStream_t stream = 0, __half* w_out = nullptr) {
  const auto v = detail::abi(p);
  detail::raise(w4_gemm_fused_mx(&v, detail::h(x), detail::h(c), M, stream, detail::h(w_out)));
}

// mxfused.cuh:291-307
inline void gemm_mma_mx(const DevicePackedWm& p, const __half* x, __half* c, int M,
                        hipStream_t stream = 0, __half* w_out = nullptr) {
  const auto v = detail::abi(p);
  detail::raise(w4_gemm_mma_mx(&v, detail::h(x), detail::h(c), M, stream, detail::h(w_out)));
}

// dispatch.cuh:36-43
inline void gemm_mx(const DevicePackedWm& p, const __half* x, __half* c, int M,
                    hipStream_t stream = 0, __half* w_out = nullptr) {
  const auto v = detail::abi(p);
  detail::raise(w4_gemm_mx(&v, detail::h(x), detail::h(c), M, stream, detail::h(w_out)));
}

// dequant.cuh:87-106.  The reference passes a cuBLAS handle; the hipBLASLt
// handle lives inside the library, so the handle type here is an empty tag.
struct BlasHandle {};
inline BlasHandle make_blas() { return BlasHandle{}; }
inline void gemm_fp16(BlasHandle, const __half* w, const __half* x, __half* c, int M, int N,
                      int K, hipStream_t stream = 0) {
  detail::raise(w4_gemm_fp16(detail::h(w), detail::h(x), detail::h(c), M, N, K, stream));
}

// kvflash.cuh:350-363
inline void attention_w4_flash(const DeviceKVW4& p, const __half* q, __half* out,
                               hipStream_t stream = 0, __half* k_out = nullptr,
                               __half* v_out = nullptr) {
  const auto v = detail::abi(p);
  detail::raise(w4_attention_w4_flash(&v, detail::h(q), detail::h(out), stream,
                                      detail::h(k_out), detail::h(v_out)));
}

// kvflash.cuh:365-384
inline void attention_fp16_flash(const __half* q, const __half* k16, const __half* v16,
                                 __half* out, int H, int S, int D, hipStream_t stream = 0) {
  detail::raise(w4_attention_fp16_flash(detail::h(q), detail::h(k16), detail::h(v16),
                                        detail::h(out), H, S, D, stream));
}

// The single-pass entry points of kvattention.cuh:226-249.  There is one
// attention kernel family here, so they run the split-S path; the sequence
// bound of the reference's shared-memory score buffer is kept so that callers
// see the same rejections.
inline void attention_fp16(const __half* q, const __half* k16, const __half* v16, __half* out,
                           int H, int S, int D, hipStream_t stream = 0) {
  if (S > KV_MAX_S) throw std::invalid_argument("kv fp16: S exceeds the shared-memory bound");
  attention_fp16_flash(q, k16, v16, out, H, S, D, stream);
}
inline void attention_w4(const DeviceKVW4& p, const __half* q, __half* out,
                         hipStream_t stream = 0, __half* k_out = nullptr,
                         __half* v_out = nullptr) {
  if (p.S > KV_MAX_S) throw std::invalid_argument("kv: S exceeds the shared-memory bound");
  attention_w4_flash(p, q, out, stream, k_out, v_out);
}

// kvflash.cuh:572-590
inline void attention_f8_flash(const DeviceKVF8& p, const __half* q, __half* out,
                               hipStream_t stream = 0, __half* k_out = nullptr,
                               __half* v_out = nullptr) {
  const auto v = detail::abi(p);
  detail::raise(w4_attention_f8_flash(&v, detail::h(q), detail::h(out), stream,
                                      detail::h(k_out), detail::h(v_out)));
}

// kvflash.cuh:725-764
inline void attention_w4_flash_paged(const DeviceKVW4& p, const int* bt, int page, int npages,
                                     const __half* q, __half* out, hipStream_t stream = 0,
                                     __half* k_out = nullptr, __half* v_out = nullptr) {
  const auto v = detail::abi(p);
  detail::raise(w4_attention_w4_flash_paged(&v, bt, page, npages, detail::h(q), detail::h(out),
                                            stream, detail::h(k_out), detail::h(v_out)));
}

// kvflash.cuh:435-457
inline void dequant_f8(const uint8_t* q, const __half* s, __half* w, int S, int D, int gs,
                       hipStream_t stream = 0) {
  detail::raise(w4_dequant_f8(q, detail::h(s), detail::h(w), S, D, gs, stream));
}

// ---- batched / grouped-query forms (additive; no reference counterpart) ------
// The views hold nseq * Hkv slabs; `group` query heads share each slab; q and
// out hold (slabs * group) * D halves, slab-major.
inline void attention_w4_flash_gqa(const DeviceKVW4& p, int group, const __half* q, __half* out,
                                   hipStream_t stream = 0, __half* k_out = nullptr,
                                   __half* v_out = nullptr) {
  const auto v = detail::abi(p);
  detail::raise(w4_attention_w4_flash_gqa(&v, group, detail::h(q), detail::h(out), stream,
                                          detail::h(k_out), detail::h(v_out)));
}

// The same call with the split-S partials in the library's built-in device array:
// no device allocation (for callers under graph capture or in loops that must not
// hipMalloc); throws std::invalid_argument when the partials exceed
// W4_NOALLOC_SCRATCH_BYTES.  Calls on one GPU share the array and must not overlap.
inline void attention_w4_flash_noalloc(const DeviceKVW4& p, int group, const __half* q,
                                       __half* out, hipStream_t stream = 0,
                                       __half* k_out = nullptr, __half* v_out = nullptr) {
  const auto v = detail::abi(p);
  detail::raise(w4_attention_w4_flash_gqa_noalloc(&v, group, detail::h(q), detail::h(out), stream,
                                                  detail::h(k_out), detail::h(v_out)));
}

inline void attention_fp16_flash_gqa(const __half* q, const __half* k16, const __half* v16,
                                     __half* out, int H, int group, int S, int D,
                                     hipStream_t stream = 0) {
  detail::raise(w4_attention_fp16_flash_gqa(detail::h(q), detail::h(k16), detail::h(v16),
                                            detail::h(out), H, group, S, D, stream));
}

// scale_mode 0: scales per (row, group) as in the reference; 1: one per slab.
inline void attention_f8_flash_gqa(const DeviceKVF8& p, int group, int scale_mode,
                                   const __half* q, __half* out, hipStream_t stream = 0,
                                   __half* k_out = nullptr, __half* v_out = nullptr) {
  const auto v = detail::abi(p);
  detail::raise(w4_attention_f8_flash_gqa(&v, group, scale_mode, detail::h(q), detail::h(out),
                                          stream, detail::h(k_out), detail::h(v_out)));
}

// One pool (p.H = Hkv slabs of npages*page rows) shared by nseq sequences, each
// with its own table of bt_stride entries.
inline void attention_w4_flash_paged_batched(const DeviceKVW4& p, const int* bt, int nseq,
                                             int bt_stride, int page, int npages, int group,
                                             const __half* q, __half* out,
                                             hipStream_t stream = 0) {
  const auto v = detail::abi(p);
  detail::raise(w4_attention_w4_flash_paged_batched(&v, bt, nseq, bt_stride, page, npages, group,
                                                    detail::h(q), detail::h(out), stream));
}

// ---- device-side quantizers ---------------------------------------------------
// The host quantizers as kernels: the views' arrays receive the bytes
// w4::quantize / quantize_mx / quantize_cache / quantize_cache_f8 would
// produce for the same values.  `status` is one device int the caller owns.
// The *_async forms only enqueue; the caller reads the status word later (bit 0
// non-finite input, bit 1 scale out of range).  The plain forms wait for the
// stream and throw what the host quantizer throws.
namespace detail {
inline void raise_status(const int* status, hipStream_t stream, const char* nonfinite,
                         const char* range) {
  int st = 0;
  hip_check(hipMemcpyAsync(&st, status, sizeof st, hipMemcpyDeviceToHost, stream), "status copy");
  hip_check(hipStreamSynchronize(stream), "status sync");
  if (st & 1) throw std::invalid_argument(nonfinite);
  if (st & 2) throw std::invalid_argument(range);
}
}  // namespace detail

// pack.hpp:64-130
inline void quantize_async(const DevicePackedW& out, const double* w, int* status,
                           hipStream_t stream = 0) {
  const auto v = detail::abi(out);
  detail::raise(w4_quantize(&v, w, status, stream));
}
inline void quantize(const DevicePackedW& out, const double* w, int* status,
                     hipStream_t stream = 0) {
  quantize_async(out, w, status, stream);
  detail::raise_status(status, stream, "quantize: non-finite input",
                       "quantize: group scale outside FP16 range");
}

// mx.hpp:71-119
inline void quantize_mx_async(const DevicePackedWm& out, const double* w, int* status,
                              hipStream_t stream = 0) {
  const auto v = detail::abi(out);
  detail::raise(w4_quantize_mx(&v, w, status, stream));
}
inline void quantize_mx(const DevicePackedWm& out, const double* w, int* status,
                        hipStream_t stream = 0) {
  quantize_mx_async(out, w, status, stream);
  detail::raise_status(status, stream, "quantize_mx: non-finite input",
                       "quantize_mx: block scale outside E8M0 range");
}

// kvcache.hpp:60-108.  k, v: H*S*D doubles, or halves with the _f16 forms (the
// append step of a decode loop, whose new rows are FP16 already).
inline void quantize_cache_async(const DeviceKVW4& out, const double* k, const double* v,
                                 int* status, hipStream_t stream = 0) {
  const auto vw = detail::abi(out);
  detail::raise(w4_quantize_cache(&vw, k, v, 0, status, stream));
}
inline void quantize_cache_f16_async(const DeviceKVW4& out, const __half* k, const __half* v,
                                     int* status, hipStream_t stream = 0) {
  const auto vw = detail::abi(out);
  detail::raise(w4_quantize_cache(&vw, k, v, 1, status, stream));
}
inline void quantize_cache(const DeviceKVW4& out, const double* k, const double* v, int* status,
                           hipStream_t stream = 0) {
  quantize_cache_async(out, k, v, status, stream);
  detail::raise_status(status, stream, "quantize: non-finite input",
                       "quantize: group scale outside FP16 range");
}

// kvfp8.hpp:70-128
inline void quantize_cache_f8_async(const DeviceKVF8& out, const double* k, const double* v,
                                    int* status, hipStream_t stream = 0) {
  const auto vw = detail::abi(out);
  detail::raise(w4_quantize_cache_f8(&vw, k, v, 0, status, stream));
}
inline void quantize_cache_f8_f16_async(const DeviceKVF8& out, const __half* k, const __half* v,
                                        int* status, hipStream_t stream = 0) {
  const auto vw = detail::abi(out);
  detail::raise(w4_quantize_cache_f8(&vw, k, v, 1, status, stream));
}
inline void quantize_cache_f8(const DeviceKVF8& out, const double* k, const double* v,
                              int* status, hipStream_t stream = 0) {
  quantize_cache_f8_async(out, k, v, status, stream);
  detail::raise_status(status, stream, "quantize_cache_f8: non-finite input",
                       "quantize_cache_f8: group scale outside FP16 range");
}

// ---- W4A4 on the scaled matrix cores (additive; the reference's MXFP4 kernels
// keep FP16 activations, mxfused.cuh:166-198,291-307) --------------------------
// Activations are quantized to MXFP4 like weights (same bytes as mx::quantize_mx
// of the FP16 values widened to FP64), then c[M,N] = X * W^T runs on packed
// operands: exact products, FP32 accumulation, FP16 output.  x.N is M.  Its
// gate is its own: rel L2 <= 1e-3 against gemm_oracle over the two dequantized
// operands.
inline void quantize_mx_f16_async(const DevicePackedWm& out, const __half* x, int* status,
                                  hipStream_t stream = 0) {
  const auto v = detail::abi(out);
  detail::raise(w4_quantize_mx_f16(&v, detail::h(x), status, stream));
}
inline void gemm_mx_w4a4(const DevicePackedWm& w, const DevicePackedWm& x, __half* c,
                         hipStream_t stream = 0) {
  const auto vw = detail::abi(w), vx = detail::abi(x);
  detail::raise(w4_gemm_mx_w4a4(&vw, &vx, detail::h(c), stream));
}

// W4A8: MXFP8 activations (include/w4/mxact.hpp), device view and entry points.
struct DeviceActMx8 {
  int M, K, B;
  const uint8_t* q;
  const uint8_t* scales;
};
inline void quantize_mx8_f16_async(const DeviceActMx8& out, const __half* x, int* status,
                                   hipStream_t stream = 0) {
  const w4_act_mx8_view v{out.M, out.K, out.B, out.q, out.scales};
  detail::raise(w4_quantize_mx8_f16(&v, detail::h(x), status, stream));
}
inline void gemm_mx_w4a8(const DevicePackedWm& w, const DeviceActMx8& x, __half* c,
                         hipStream_t stream = 0) {
  const auto vw = detail::abi(w);
  const w4_act_mx8_view vx{x.M, x.K, x.B, x.q, x.scales};
  detail::raise(w4_gemm_mx_w4a8(&vw, &vx, detail::h(c), stream));
}

}  // namespace w4::gpu
