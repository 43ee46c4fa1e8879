// Materialising dequant kernels: packed W4 / MXFP4 weights and FP8 cache rows
// to FP16 in HBM.  They are the first pass of the two-pass baseline and the
// bitwise gate for the dequant arithmetic; the fused kernels never call them.
//
// One lane expands one packed word (8 weights, or 4 FP8 bytes) and writes it
// with a single 16-byte (8-byte) store when the row layout allows it, so a
// wave reads 256 contiguous bytes and writes 1 KiB contiguous.
#include "dq.cuh"
#include "kernels.h"

namespace w4k {

template <int MX, bool VEC>
__global__ __launch_bounds__(256) void dequant_words(WView p, w4_half* __restrict__ w,
                                                     long long total, int wpr) {
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= total) return;
  const int n = (int)(idx / wpr);
  const int wi = (int)(idx - (long long)n * wpr);
  const int k0 = wi * 8;
  const uint32_t qw = p.q[idx];
  h2 d[4], nat[4];
  if (MX) {
    dq_mx(qw, mx_scale(((const uint8_t*)p.scales)[(size_t)n * p.B + (k0 >> 5)]), nat);
  } else {
    const int g = k0 / p.gs;
    const uint16_t sb = ((const uint16_t*)p.scales)[(size_t)n * p.G + g];
    const int z = p.symmetric
                      ? 8
                      : (int)((p.zeros[(size_t)n * words(p.G) + (g >> 3)] >> (4 * (g & 7))) & 0xF);
    dq_w4(qw, w4_group(sb, z), d);
    to_natural(d, nat);
  }
  uint16_t* out = w + (size_t)n * p.K + k0;
  if (VEC) {
    *(u4*)out = u4{as_u32(nat[0]), as_u32(nat[1]), as_u32(nat[2]), as_u32(nat[3])};
  } else {
#pragma unroll
    for (int j = 0; j < 8; ++j)
      if (k0 + j < p.K) {
        const uint32_t pair = as_u32(nat[j >> 1]);
        out[j] = (uint16_t)((j & 1) ? pair >> 16 : pair & 0xFFFFu);
      }
  }
}

hipError_t launch_dequant(const WView& v, w4_half* w, hipStream_t s) {
  const int wpr = words(v.K);
  const long long total = (long long)v.N * wpr;
  const unsigned grid = (unsigned)((total + 255) / 256);
  const bool vec = (v.K % 8 == 0) && (((uintptr_t)w & 15) == 0);
  if (v.mx) {
    if (vec) dequant_words<1, true><<<grid, 256, 0, s>>>(v, w, total, wpr);
    else dequant_words<1, false><<<grid, 256, 0, s>>>(v, w, total, wpr);
  } else {
    if (vec) dequant_words<0, true><<<grid, 256, 0, s>>>(v, w, total, wpr);
    else dequant_words<0, false><<<grid, 256, 0, s>>>(v, w, total, wpr);
  }
  return hipGetLastError();
}

// FP8 rows: one lane per 4-byte word (D % 4 == 0 and a 4-byte-aligned base are
// entry contracts), scale index d0 / gs within the row.
__global__ __launch_bounds__(256) void dequant_f8_words(const uint8_t* __restrict__ q,
                                                        const w4_half* __restrict__ sc,
                                                        w4_half* __restrict__ w,
                                                        long long total, int wpr, int D,
                                                        int gs, int G, bool vec) {
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= total) return;
  const long long t = idx / wpr;
  const int d0 = 4 * (int)(idx - t * wpr);
  const uint32_t qw = ((const uint32_t*)q)[idx];
  h2 d[2], nat[2];
  dq_f8(qw, splat_bits(sc[t * G + d0 / gs]), d);
  to_natural_f8(d, nat);
  uint16_t* out = w + t * D + d0;
  if (vec) {
    *(u2*)out = u2{as_u32(nat[0]), as_u32(nat[1])};
  } else {
    out[0] = (uint16_t)(as_u32(nat[0]) & 0xFFFFu);
    out[1] = (uint16_t)(as_u32(nat[0]) >> 16);
    out[2] = (uint16_t)(as_u32(nat[1]) & 0xFFFFu);
    out[3] = (uint16_t)(as_u32(nat[1]) >> 16);
  }
}

hipError_t launch_dequant_f8(const uint8_t* q, const w4_half* sc, w4_half* w, int S,
                             int D, int gs, hipStream_t s) {
  const int wpr = D / 4;
  const long long total = (long long)S * wpr;
  const int G = (D + gs - 1) / gs;
  const bool vec = ((uintptr_t)w & 7) == 0;
  dequant_f8_words<<<(unsigned)((total + 255) / 256), 256, 0, s>>>(q, sc, w, total, wpr,
                                                                   D, gs, G, vec);
  return hipGetLastError();
}

}  // namespace w4k
