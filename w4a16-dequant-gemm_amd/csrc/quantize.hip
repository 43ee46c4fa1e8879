// Device-side quantizers: the host quantizers of the packed formats as gfx950
// kernels, producing the same bytes.
//
//   rows of W4 codes (weights and KV-cache rows) ... pack.hpp:64-130, kvcache.hpp:60-108
//   rows of E4M3 bytes (FP8 KV cache) ............... kvfp8.hpp:70-128
//   rows of MXFP4 codes ............................. mx.hpp:71-119
//
// Bit identity with the host comes from doing the same IEEE operations in the
// same order: min/max and the step in FP64, the step rounded FP64 -> FP32 ->
// FP16 in two hardware conversions (both round to nearest even, FP16
// subnormals kept), every element divided in FP64 by the stored scale, and
// round-half-away-from-zero done on the exact fraction.  The MXFP4 block
// exponent is the smallest e with amax <= 6 * 2^e, which is what the host's
// ceil(log2(amax / 6)) followed by its upward fix-up loop evaluates to; here
// it is read off the exponent field and settled by one exact comparison.
//
// The kernels are memory-bound streams: one thread per packed word (8 elements
// in, 4 or 8 bytes out), group extrema combined through LDS.  Conditions the
// host reports by throwing (non-finite input, scale outside the FP16 / E8M0
// range) are OR-ed into a caller-provided status word: bit 0 non-finite input,
// bit 1 scale out of range.  Outputs are unspecified when it ends non-zero.
#include <float.h>

#include "dq.cuh"
#include "kernels.h"

namespace w4k {
namespace {

constexpr int QT = 256;  // threads per workgroup

__global__ void fill_words_kernel(uint32_t* p, long long n, uint32_t value) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = value;
}

enum { QM_SYM = 0, QM_ASYM = 1, QM_F8 = 2 };

// Up to two independent jobs of the same shape in one launch (the K and the V
// side of a cache): blockIdx.y picks the side.
template <typename T>
struct Sides {
  const T* src[2];
  uint32_t* q32[2];
  uint8_t* q8[2];
  uint16_t* scales[2];
  uint32_t* zeros[2];
};

// lround() for |v| far below 2^52: the fraction v - trunc(v) is exact.
__device__ __forceinline__ long round_half_away(double v) {
  double t = trunc(v);
  const double frac = fabs(v - t);
  t = fmin(fmax(t, -1.0e12), 1.0e12);
  long r = (long)t;
  if (frac >= 0.5) r += v < 0.0 ? -1 : 1;
  return r;
}

__device__ __forceinline__ int clamp_code(long v) { return (int)(v < 0 ? 0 : (v > 15 ? 15 : v)); }

__device__ __forceinline__ bool finite(double x) { return fabs(x) <= DBL_MAX; }

// kvfp8.hpp:48-53 (the encoder of quantize_cache_f8): round to nearest even on
// the E4M3 grid, saturate at 448, NaN -> 0x7F.
__device__ __forceinline__ uint32_t encode_e4m3(float x) {
  const uint32_t bits = __builtin_bit_cast(uint32_t, x);
  const uint32_t sign = (bits >> 24) & 0x80u;
  const float a = fabsf(x);
  if (a != a) return sign | 0x7Fu;
  if (a >= 448.0f) return sign | 0x7Eu;
  int ex = (int)((bits >> 23) & 0xFFu) - 127;
  if (ex < -6) ex = -6;
  // a * 2^(3 - ex) is exact; one rint is the rounding (0..16 steps)
  const int steps = (int)rintf(a * __builtin_bit_cast(float, (uint32_t)(130 - ex) << 23));
  const int code = (ex == -6 && steps < 8) ? steps : (ex + 7) * 8 + (steps - 8);
  return sign | (uint32_t)(code > 0x7E ? 0x7E : code);
}

// encode_e4m3(v / s) for FP16-representable v and s without the division.  x = v * (1 / s)
// is within 2^-22 (relative) of the exact quotient q.  q has 11-bit numerator and
// denominator, so it is either exactly on a midpoint of the E4M3 grid (odd multiples
// of half a step, at most 31) or at least 2^-16 (relative) away from every one: if x
// is within 2^-20 of a midpoint, q is that midpoint and the tie goes to the even code;
// otherwise x and q round alike.  (The host rounds the FP64 quotient to FP32 first,
// which for the same reason never moves it onto or across a midpoint.)
__device__ __forceinline__ uint32_t encode_e4m3_quotient(float v, float rs) {
  const float x = v * rs;
  const uint32_t sign = (__builtin_bit_cast(uint32_t, x) >> 24) & 0x80u;
  // straight-line code (as early returns per element the compiler made 16 divergent
  // regions per thread): saturation is the grid's own top, 448 = 14 steps of 2^5
  const float a = fminf(fabsf(x), 448.0f);
  int ex = (int)((__builtin_bit_cast(uint32_t, a) >> 23) & 0xFFu) - 127;
  ex = ex < -6 ? -6 : ex;
  const float y = a * __builtin_bit_cast(float, (uint32_t)(130 - ex) << 23);  // exact; 0 .. 16 steps
  const float f = floorf(y);
  const float d = fabsf((y - f) - 0.5f);  // distance from the midpoint, exact
  float r = rintf(y);
  r = d < y * 0x1p-20f ? f + (float)((int)f & 1) : r;
  const int steps = (int)r;
  int code = (ex + 7) * 8 + (steps - 8);  // with ex = -6 this is `steps` itself, subnormal or not
  code = code > 0x7E ? 0x7E : code;
  code = x != x ? 0x7F : code;
  return sign | (uint32_t)code;
}

__device__ __forceinline__ int pow2_at_least(int n) {
  int p = 1;
  while (p < n) p <<= 1;
  return p;
}

// One workgroup quantizes QT / tpg consecutive (row, group) pairs, tpg =
// min(gs / 8, QT) threads each; a thread owns whole packed words.  T is the
// source element type (double or _Float16).
template <typename T, int MODE>
__global__ __launch_bounds__(QT) void quantize_rows_kernel(
    const Sides<T> sd, long long rows, int K, int gs, int G, int* __restrict__ status) {
  const T* __restrict__ src = sd.src[blockIdx.y];
  uint32_t* __restrict__ q32 = sd.q32[blockIdx.y];
  uint8_t* __restrict__ q8 = sd.q8[blockIdx.y];
  uint16_t* __restrict__ scales = sd.scales[blockIdx.y];
  uint32_t* __restrict__ zeros = sd.zeros[blockIdx.y];
  __shared__ double s_lo[QT], s_hi[QT];
  __shared__ float s_scale[QT];
  __shared__ int s_zero[QT];

  const int wpg = gs >> 3;
  const int tpg = wpg < QT ? wpg : QT;
  const int gpb = QT / tpg;
  const int t = threadIdx.x;
  const int lg = t / tpg, li = t - lg * tpg;
  const long long gid = (long long)blockIdx.x * gpb + lg;
  const bool live = lg < gpb && gid < rows * G;
  long long row = 0;
  int g = 0;
  if (live) {
    row = gid / G;
    g = (int)(gid - row * G);
  }
  const int k0 = g * gs;
  const int len = live ? (gs < K - k0 ? gs : K - k0) : 0;
  const int nw = (len + 7) >> 3;
  const T* base = src + row * (long long)K + k0;

  // extrema of this thread's words; the first word stays in registers
  double lo = INFINITY, hi = -INFINITY;
  double first[8];
  bool bad = false;
#pragma unroll
  for (int j = 0; j < 8; ++j) first[j] = 0.0;
  for (int wi = li; wi < nw; wi += tpg) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int e = wi * 8 + j;
      if (e < len) {
        const double x = (double)base[e];
        bad |= !finite(x);
        lo = fmin(lo, x);
        hi = fmax(hi, x);
        if (wi == li) first[j] = x;
      }
    }
  }
  if (bad) atomicOr(status, 1);

  s_lo[t] = lo;
  s_hi[t] = hi;
  __syncthreads();
  for (int s = pow2_at_least(tpg) >> 1; s > 0; s >>= 1) {
    if (li < s && li + s < tpg) {
      s_lo[t] = fmin(s_lo[t], s_lo[t + s]);
      s_hi[t] = fmax(s_hi[t], s_hi[t + s]);
    }
    __syncthreads();
  }

  if (live && li == 0) {
    lo = s_lo[t];
    hi = s_hi[t];
    double step = 1.0;
    bool has_signal;
    if (MODE == QM_ASYM) {
      lo = fmin(lo, 0.0);
      hi = fmax(hi, 0.0);
      if (hi > lo) step = (hi - lo) / 15.0;
      has_signal = hi != lo;
    } else {
      const double amax = fmax(fabs(lo), fabs(hi));
      if (amax > 0.0) step = amax / (MODE == QM_F8 ? 448.0 : 7.0);
      has_signal = amax > 0.0;
    }
    float step_f = (float)step;
    // the host rounds in two steps; keep the compiler from folding the two
    // conversions into one FP64 -> FP16 rounding, which differs on ties
    asm volatile("" : "+v"(step_f));
    const _Float16 sh = (_Float16)step_f;
    const float sf = (float)sh;
    if (!(fabsf(sf) <= FLT_MAX) || (sf == 0.0f && has_signal)) atomicOr(status, 2);
    int zero = 8;
    if (MODE == QM_ASYM) {
      zero = clamp_code(round_half_away(-lo / (double)sf));
      atomicOr(zeros + row * (long long)words(G) + (g >> 3), (uint32_t)zero << (4 * (g & 7)));
    }
    scales[gid] = __builtin_bit_cast(uint16_t, sh);
    s_scale[lg] = sf;
    s_zero[lg] = zero;
  }
  __syncthreads();
  if (!live) return;

  const double sf = (double)s_scale[lg];
  const int zero = s_zero[lg];
  for (int wi = li; wi < nw; wi += tpg) {
    double v[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int e = wi * 8 + j;
      v[j] = wi == li ? first[j] : (e < len ? (double)base[e] : 0.0);
    }
    if (MODE == QM_F8) {
      uint8_t* dst = q8 + row * (long long)K + k0 + wi * 8;
      uint32_t b[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) b[j] = encode_e4m3((float)(v[j] / sf));
      if (wi * 8 + 8 <= len && ((uintptr_t)dst & 7) == 0) {
        u2 out;
        out[0] = b[0] | (b[1] << 8) | (b[2] << 16) | (b[3] << 24);
        out[1] = b[4] | (b[5] << 8) | (b[6] << 16) | (b[7] << 24);
        *(u2*)dst = out;
      } else {
#pragma unroll
        for (int j = 0; j < 8; ++j)
          if (wi * 8 + j < len) dst[j] = (uint8_t)b[j];
      }
    } else {
      uint32_t word = 0;
#pragma unroll
      for (int j = 0; j < 8; ++j)
        if (wi * 8 + j < len)
          word |= (uint32_t)clamp_code(round_half_away(v[j] / sf) + zero) << (4 * j);
      q32[row * (long long)words(K) + (k0 >> 3) + wi] = word;
    }
  }
}

// Arithmetic type of the per-element quotient.  FP64 sources divide in FP64 as
// the host does.  FP16 sources divide in FP32: value and scale have 11-bit
// significands, so the exact quotient is either on a rounding boundary (k + 1/2
// for the codes, a 25-bit midpoint for the FP32 quotient the E4M3 encoder
// takes) or at least 2^-14 (2^-36 relative) away from it -- far more than the
// FP32 (FP64) rounding error -- and the correctly rounded FP32 quotient gives
// the code the host's FP64 quotient gives.
template <typename T> struct Quot { typedef double type; };
template <> struct Quot<_Float16> { typedef float type; };

__device__ __forceinline__ int round_half_away_small(float v) {
  float t = truncf(v);
  const float frac = fabsf(v - t);
  t = fminf(fmaxf(t, -1.0e6f), 1.0e6f);
  int r = (int)t;
  if (frac >= 0.5f) r += v < 0.0f ? -1 : 1;
  return r;
}
__device__ __forceinline__ int round_half_away_small(double v) { return (int)round_half_away(v); }

// round_half_away(v / sf) for FP16-representable v and sf > 0 without the division: a
// candidate from v * (1 / sf) (a few ulp off, so within one of the answer while
// |v / sf| <= 64; beyond that every code saturates), then the two tests that define the
// answer, v - (c -+ 1/2) sf against zero, each one fused multiply-add whose sign is
// the exact sign (it rounds an exact real, and a nonzero difference of multiples of
// 2^-25 cannot underflow).  A third fewer vector instructions than the correctly
// rounded quotient plus its rounding, in a kernel that is bound by them.
__device__ __forceinline__ int round_quotient_half_away(float v, float sf, float rsf) {
  const float a = fabsf(v);  // half away from zero: round the magnitude half up, restore the sign
  const float t = fminf(a * rsf, 64.0f);
  const float c = rintf(t);
  const float lo = fmaf(0.5f - c, sf, a);   // |v| - (c - 1/2) sf
  const float hi = fmaf(-0.5f - c, sf, a);  // |v| - (c + 1/2) sf
  int m = (int)c;
  m -= lo < 0.0f ? 1 : 0;  // (straight-line code: as branches this was slower than the division)
  m += hi >= 0.0f ? 1 : 0;
  return v < 0.0f ? -m : m;
}

__device__ __forceinline__ void load8(const double* p, double v[8]) {
  typedef double d2 __attribute__((ext_vector_type(2)));
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const d2 x = ((const d2*)p)[i];
    v[2 * i] = x[0];
    v[2 * i + 1] = x[1];
  }
}
__device__ __forceinline__ void load8(const _Float16* p, float v[8]) {
  const h8 x = *(const h8*)p;
#pragma unroll
  for (int i = 0; i < 8; ++i) v[i] = (float)x[i];
}

// Whole rows of full groups whose word count is a power of two up to 64: a
// thread owns packed word `w` of the flattened (row, k) space, the gs / 8 lanes
// of a group combine their extrema with lane exchanges and every lane derives
// the group's scale itself -- no LDS round trip, fully coalesced 16-byte loads.
// ZPACK: zero-point words are assembled through LDS (G and the groups per
// workgroup both multiples of 8); otherwise nibbles are OR-ed in atomically.
template <typename T, int MODE, bool ZPACK>
__global__ __launch_bounds__(QT) void quantize_rows_fast_kernel(
    const Sides<T> sd, long long nwords, int wpg, int wpg_shift, int G, int* __restrict__ status) {
  const T* __restrict__ src = sd.src[blockIdx.y];
  uint32_t* __restrict__ q32 = sd.q32[blockIdx.y];
  uint8_t* __restrict__ q8 = sd.q8[blockIdx.y];
  uint16_t* __restrict__ scales = sd.scales[blockIdx.y];
  uint32_t* __restrict__ zeros = sd.zeros[blockIdx.y];
  typedef typename Quot<T>::type A;
  __shared__ int s_zero[QT];
  const int t = threadIdx.x;
  const long long w = (long long)blockIdx.x * QT + t;
  const bool live = w < nwords;
  A v[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) v[j] = (A)0;
  if (live) load8(src + w * 8, v);
  A lo = v[0], hi = v[0];
  bool bad = false;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    if (sizeof(T) == 2) bad |= !(fabsf((float)v[j]) <= 65504.0f);
    else bad |= !(fabs((double)v[j]) <= DBL_MAX);
    lo = v[j] < lo ? v[j] : lo;
    hi = v[j] > hi ? v[j] : hi;
  }
  if (bad) atomicOr(status, 1);
  for (int m = 1; m < wpg; m <<= 1) {
    const A olo = __shfl_xor(lo, m), ohi = __shfl_xor(hi, m);
    lo = olo < lo ? olo : lo;
    hi = ohi > hi ? ohi : hi;
  }
  // Scale of the group, in every lane.  The step goes FP64 -> FP32 -> FP16 on the
  // host.  For FP16 sources without zero-points the FP32 step is amax / 7 (/ 448)
  // of an 11-bit amax: its binary expansion is periodic with period 3, so it is
  // never within an FP64 rounding error of an FP32 midpoint and one correctly
  // rounded FP32 division gives the same FP32 value as the two-step rounding.
  float step_f;
  bool has_signal;
  double dlo = (double)lo, dhi = (double)hi;
  if (MODE == QM_ASYM) {
    dlo = fmin(dlo, 0.0);
    dhi = fmax(dhi, 0.0);
    step_f = (float)(dhi > dlo ? (dhi - dlo) / 15.0 : 1.0);
    has_signal = dhi != dlo;
  } else if (sizeof(T) == 2) {
    const float amax = fmaxf(fabsf((float)lo), fabsf((float)hi));
    step_f = amax > 0.0f ? amax / (MODE == QM_F8 ? 448.0f : 7.0f) : 1.0f;
    has_signal = amax > 0.0f;
  } else {
    const double amax = fmax(fabs(dlo), fabs(dhi));
    step_f = (float)(amax > 0.0 ? amax / (MODE == QM_F8 ? 448.0 : 7.0) : 1.0);
    has_signal = amax > 0.0;
  }
  asm volatile("" : "+v"(step_f));  // keep the FP32 and FP16 roundings separate
  const _Float16 sh = (_Float16)step_f;
  const float sf = (float)sh;
  int zero = 8;
  if (MODE == QM_ASYM) zero = clamp_code(round_half_away(-dlo / (double)sf));
  const bool leader = live && (t & (wpg - 1)) == 0;
  const long long gid = w >> wpg_shift;
  if (leader) {
    if (!(fabsf(sf) <= FLT_MAX) || (sf == 0.0f && has_signal)) atomicOr(status, 2);
    scales[gid] = __builtin_bit_cast(uint16_t, sh);
    if (MODE == QM_ASYM && !ZPACK) {
      const long long row = gid / G;
      const int g = (int)(gid - row * G);
      atomicOr(zeros + row * (long long)words(G) + (g >> 3), (uint32_t)zero << (4 * (g & 7)));
    }
  }
  if (MODE == QM_ASYM && ZPACK) {
    if ((t & (wpg - 1)) == 0) s_zero[t >> wpg_shift] = zero;
    __syncthreads();
    const int gpb = QT >> wpg_shift;
    const long long zw = ((long long)blockIdx.x * gpb >> 3) + t;
    if (t < (gpb >> 3) && zw * 8 * wpg < nwords) {
      uint32_t word = 0;
#pragma unroll
      for (int j = 0; j < 8; ++j) word |= (uint32_t)s_zero[t * 8 + j] << (4 * j);
      zeros[zw] = word;
    }
  }
  if (!live) return;
  const A sfa = (A)sf;
  if (MODE == QM_F8) {
    uint32_t b[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      if constexpr (sizeof(T) == 2) b[j] = encode_e4m3_quotient((float)v[j], __builtin_amdgcn_rcpf(sf));
      else b[j] = encode_e4m3((float)(v[j] / sfa));
    }
    u2 out;
    out[0] = b[0] | (b[1] << 8) | (b[2] << 16) | (b[3] << 24);
    out[1] = b[4] | (b[5] << 8) | (b[6] << 16) | (b[7] << 24);
    *(u2*)(q8 + w * 8) = out;
  } else {
    uint32_t word = 0;
    const float rsf = __builtin_amdgcn_rcpf(sf);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      int c;
      if constexpr (sizeof(T) == 2) c = round_quotient_half_away((float)v[j], sf, rsf) + zero;
      else c = round_half_away_small(v[j] / sfa) + zero;
      word |= (uint32_t)(c < 0 ? 0 : (c > 15 ? 15 : c)) << (4 * j);
    }
    q32[w] = word;
  }
}

// mx.hpp:91-101 in closed form: the smallest e with amax <= TOP * 2^e, TOP the
// largest magnitude of the element type (6 for E2M1, 448 for E4M3).  With amax in
// [2^p, 2^(p+1)) the answer lies within two steps of p - ilogb(TOP).
template <int TOP>
__device__ __forceinline__ int mx_exponent(double amax, bool* out_of_range) {
  if (!(amax > 0.0)) return 0;
  if (amax <= (double)TOP * 0x1p-127) return -127;
  const int p = (int)((__builtin_bit_cast(uint64_t, amax) >> 52) & 0x7FFu) - 1023;
  int e = p - (TOP == 6 ? 2 : 9);  // TOP * 2^(e - 1) < 2^p <= amax
  if (amax > (double)TOP * ldexp(1.0, e)) ++e;
  if (amax > (double)TOP * ldexp(1.0, e)) ++e;
  if (e > 127) {
    *out_of_range = true;
    e = 127;
  }
  return e;
}

// mx.hpp:103-108: index of the nearest E2M1 magnitude, the lower one on ties.
// (In FP32 for FP16 sources: the scaled value has 11 significant bits, so every
// difference below is exact and a tie is a tie.)
template <typename A>
__device__ __forceinline__ int nearest_e2m1(A a) {
  const A mags[8] = {(A)0.0, (A)0.5, (A)1.0, (A)1.5, (A)2.0, (A)3.0, (A)4.0, (A)6.0};
  int best = 0;
  A dbest = a;
#pragma unroll
  for (int i = 1; i < 8; ++i) {
    const A d = __builtin_elementwise_abs(mags[i] - a);
    if (d < dbest) {
      best = i;
      dbest = d;
    }
  }
  return best;
}

// Four threads per 32-element block, eight elements each: one packed word of
// E2M1 codes, or (F8: the MXFP8 activation format, no host counterpart in the
// reference; same block rule with 448 in place of 6) eight E4M3 bytes.
template <typename T, bool FULL, bool F8>
__global__ __launch_bounds__(QT) void quantize_mx_kernel(const T* __restrict__ src,
                                                         long long rows, int K, int B,
                                                         uint32_t* __restrict__ q,
                                                         uint8_t* __restrict__ q8,
                                                         uint8_t* __restrict__ scales,
                                                         int* __restrict__ status) {
  const long long id = (long long)blockIdx.x * QT + threadIdx.x;
  const long long blk = id >> 2;
  const int j4 = (int)(id & 3);
  const bool live = blk < rows * B;
  long long row = 0;
  int b = 0;
  if (live) {
    row = blk / B;
    b = (int)(blk - row * B);
  }
  const int k0 = b * 32 + j4 * 8;
  const int n = live ? (K - k0 < 0 ? 0 : (K - k0 > 8 ? 8 : K - k0)) : 0;
  const T* base = src + row * (long long)K + k0;
  // FP16 sources work in FP32: scaling by a power of two is exact, and so is
  // everything the encoders do with an 11-bit significand
  typedef typename Quot<T>::type A;
  A v[8];
  A amax = (A)0;
  bool bad = false;
  if constexpr (FULL) {  // K a multiple of 8 and 16-byte aligned rows: four 16-byte loads
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = (A)0;
    if (n) load8(base, v);
  } else {
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = j < n ? (A)base[j] : (A)0;
  }
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const A av = v[j] < (A)0 ? -v[j] : v[j];
    bad |= !(av <= (A)(sizeof(T) == 2 ? 65504.0 : DBL_MAX));
    amax = av > amax ? av : amax;
  }
  if (bad) atomicOr(status, 1);
  {
    const A o1 = __shfl_xor(amax, 1);
    amax = o1 > amax ? o1 : amax;
    const A o2 = __shfl_xor(amax, 2);
    amax = o2 > amax ? o2 : amax;
  }
  bool range = false;
  const int e = mx_exponent<F8 ? 448 : 6>((double)amax, &range);
  if (range && j4 == 0) atomicOr(status, 2);
  if (n == 0) return;
  A u[8];  // v / 2^e
  if constexpr (sizeof(T) == 2) {
#pragma unroll
    for (int j = 0; j < 8; ++j) u[j] = ldexpf(v[j], -e);
  } else {
    // |e| <= 127, so 2^-e is a normal double and v * 2^-e is the same real number
    // as v / 2^e, rounded the same way: the host's quotient without the division
    const double inv = ldexp(1.0, -e);
#pragma unroll
    for (int j = 0; j < 8; ++j) u[j] = v[j] * inv;
  }
  if (F8) {
    uint8_t* dst = q8 + row * (long long)K + k0;
    uint32_t c[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) c[j] = encode_e4m3((float)u[j]);
    if (n == 8 && ((uintptr_t)dst & 7) == 0) {
      u2 out;
      out[0] = c[0] | (c[1] << 8) | (c[2] << 16) | (c[3] << 24);
      out[1] = c[4] | (c[5] << 8) | (c[6] << 16) | (c[7] << 24);
      *(u2*)dst = out;
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j)
        if (j < n) dst[j] = (uint8_t)c[j];
    }
  } else {
    uint32_t word = 0;
#pragma unroll
    for (int j = 0; j < 8; ++j)
      if (j < n) {
        const uint32_t code = (__builtin_signbit(u[j]) ? 8u : 0u) |
                              (uint32_t)nearest_e2m1<A>(u[j] < (A)0 ? -u[j] : u[j]);
        word |= code << (4 * j);
      }
    q[row * (long long)words(K) + b * 4 + j4] = word;
  }
  if (j4 == 0) scales[blk] = (uint8_t)(e + 127);
}

template <typename T, int MODE>
hipError_t launch_rows_t(const Sides<T>& sd, int nsides, long long rows, int K, int gs,
                         int* status, hipStream_t s) {
  const int G = (K + gs - 1) / gs;
  const int wpg = gs >> 3, tpg = wpg < QT ? wpg : QT, gpb = QT / tpg;
  const bool pow2 = (wpg & (wpg - 1)) == 0;
  bool aligned = true;
  for (int i = 0; i < nsides; ++i)
    aligned = aligned && ((uintptr_t)sd.src[i] & 15) == 0 &&
              (MODE != QM_F8 || ((uintptr_t)sd.q8[i] & 7) == 0);
  const bool fast = pow2 && wpg <= 64 && K % gs == 0 && aligned;
  const bool zpack = fast && MODE == QM_ASYM && G % 8 == 0 && (QT / wpg) % 8 == 0;
  if (MODE == QM_ASYM && !zpack) {
    // zero-points are OR-ed in nibble by nibble
    const long long nz = rows * words(G);
    for (int i = 0; i < nsides; ++i)
      fill_words_kernel<<<dim3((unsigned)((nz + 255) / 256)), dim3(256), 0, s>>>(sd.zeros[i], nz, 0u);
  }
  if (fast) {
    const long long nwords = rows * (K >> 3);
    const long long nb = (nwords + QT - 1) / QT;
    if (nb > 0x7FFFFFFFLL) return hipErrorInvalidConfiguration;
    const int shift = __builtin_ctz(wpg);
    const dim3 grid((unsigned)nb, (unsigned)nsides);
    if (zpack)
      quantize_rows_fast_kernel<T, MODE, true><<<grid, dim3(QT), 0, s>>>(sd, nwords, wpg, shift, G,
                                                                        status);
    else
      quantize_rows_fast_kernel<T, MODE, false><<<grid, dim3(QT), 0, s>>>(sd, nwords, wpg, shift,
                                                                         G, status);
    return hipGetLastError();
  }
  const long long blocks = (rows * G + gpb - 1) / gpb;
  if (blocks > 0x7FFFFFFFLL) return hipErrorInvalidConfiguration;
  quantize_rows_kernel<T, MODE><<<dim3((unsigned)blocks, (unsigned)nsides), dim3(QT), 0, s>>>(
      sd, rows, K, gs, G, status);
  return hipGetLastError();
}

template <typename T>
hipError_t launch_rows(int mode, const QuantSide* sides, int nsides, long long rows, int K, int gs,
                       int* status, hipStream_t s) {
  Sides<T> sd{};
  for (int i = 0; i < nsides; ++i) {
    sd.src[i] = (const T*)sides[i].src;
    sd.q32[i] = sides[i].q32;
    sd.q8[i] = sides[i].q8;
    sd.scales[i] = sides[i].scales;
    sd.zeros[i] = sides[i].zeros;
  }
  if (mode == QM_SYM) return launch_rows_t<T, QM_SYM>(sd, nsides, rows, K, gs, status, s);
  if (mode == QM_ASYM) return launch_rows_t<T, QM_ASYM>(sd, nsides, rows, K, gs, status, s);
  return launch_rows_t<T, QM_F8>(sd, nsides, rows, K, gs, status, s);
}

}  // namespace

hipError_t launch_fill_words(uint32_t* p, long long n, uint32_t value, hipStream_t s) {
  fill_words_kernel<<<dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s>>>(p, n, value);
  return hipGetLastError();
}

hipError_t launch_quantize_rows(int mode, const QuantSide* sides, int nsides, int src_f16,
                                long long rows, int K, int gs, int* status, hipStream_t s) {
  return src_f16 ? launch_rows<_Float16>(mode, sides, nsides, rows, K, gs, status, s)
                 : launch_rows<double>(mode, sides, nsides, rows, K, gs, status, s);
}

hipError_t launch_quantize_mx(const void* src, int src_f16, long long rows, int K, uint32_t* q,
                              uint8_t* scales, int* status, hipStream_t s) {
  const int B = (K + 31) / 32;
  const long long blocks = (rows * B * 4 + QT - 1) / QT;
  if (blocks > 0x7FFFFFFFLL) return hipErrorInvalidConfiguration;
  const dim3 grid((unsigned)blocks), block(QT);
  const bool vec = K % 8 == 0 && ((uintptr_t)src & 15) == 0;
  if (src_f16 && vec)
    quantize_mx_kernel<_Float16, true, false><<<grid, block, 0, s>>>((const _Float16*)src, rows, K,
                                                                    B, q, nullptr, scales, status);
  else if (src_f16)
    quantize_mx_kernel<_Float16, false, false><<<grid, block, 0, s>>>((const _Float16*)src, rows, K,
                                                                     B, q, nullptr, scales, status);
  else if (K % 8 == 0 && ((uintptr_t)src & 15) == 0)
    quantize_mx_kernel<double, true, false><<<grid, block, 0, s>>>((const double*)src, rows, K, B,
                                                                  q, nullptr, scales, status);
  else
    quantize_mx_kernel<double, false, false><<<grid, block, 0, s>>>((const double*)src, rows, K, B,
                                                                   q, nullptr, scales, status);
  return hipGetLastError();
}

hipError_t launch_quantize_mx8(const void* src, int src_f16, long long rows, int K, uint8_t* q,
                               uint8_t* scales, int* status, hipStream_t s) {
  const int B = (K + 31) / 32;
  const long long blocks = (rows * B * 4 + QT - 1) / QT;
  if (blocks > 0x7FFFFFFFLL) return hipErrorInvalidConfiguration;
  const dim3 grid((unsigned)blocks), block(QT);
  if (src_f16 && K % 8 == 0 && ((uintptr_t)src & 15) == 0)
    quantize_mx_kernel<_Float16, true, true><<<grid, block, 0, s>>>((const _Float16*)src, rows, K,
                                                                   B, nullptr, q, scales, status);
  else if (src_f16)
    quantize_mx_kernel<_Float16, false, true><<<grid, block, 0, s>>>((const _Float16*)src, rows, K,
                                                                    B, nullptr, q, scales, status);
  else
    quantize_mx_kernel<double, false, true><<<grid, block, 0, s>>>((const double*)src, rows, K, B,
                                                                  nullptr, q, scales, status);
  return hipGetLastError();
}

}  // namespace w4k
