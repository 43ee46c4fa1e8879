// Register-level dequantisation steps shared by every gfx950 kernel.
//
// A packed word (8 four-bit codes along K) is expanded in VGPRs to four
// packed-half registers.  All arithmetic stays in FP16 and is bit-identical to
// the host step RNE_half(float(scale) * value):
//   * the code value (q - z, an E2M1 magnitude, an E4M3 magnitude) is formed
//     exactly in FP16;
//   * the scale has an 11-bit significand and the value at most 4 significant
//     bits, so the exact product fits FP32 and v_pk_mul_f16 performs the same
//     single round-to-nearest-even (FP16 denormals are enabled on gfx950).
// The pairs come out "strided": register i holds elements (i, i+4) of the
// word, which is what two mask-and-or instructions per pair give for free.
// to_natural() re-pairs them as (0,1),(2,3),(4,5),(6,7) with v_perm_b32.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace w4k {

typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef _Float16 h4 __attribute__((ext_vector_type(4)));
typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef uint32_t u4 __attribute__((ext_vector_type(4)));
typedef uint32_t u2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ h2 as_h2(uint32_t u) { return __builtin_bit_cast(h2, u); }
__device__ __forceinline__ uint32_t as_u32(h2 h) { return __builtin_bit_cast(uint32_t, h); }
__device__ __forceinline__ h2 splat(_Float16 v) { return h2{v, v}; }
__device__ __forceinline__ h2 splat_bits(uint32_t b16) { return as_h2(b16 * 0x00010001u); }

__host__ __device__ __forceinline__ int words(int n) { return (n + 7) >> 3; }

// ---- W4 affine codes ------------------------------------------------------
// Per group: scale (FP16) and zero-point z (8 when symmetric).
struct W4Group {
  h2 s;    // scale, both lanes
  h2 zlo;  // 1024 + z
  h2 zhi;  // 64 + z
};

__device__ __forceinline__ W4Group w4_group(uint16_t scale_bits, int z) {
  W4Group g;
  g.s = splat_bits(scale_bits);
  g.zlo = splat_bits(0x6400u | (uint32_t)z);         // 1024 + z, ulp 1
  g.zhi = splat_bits(0x5400u | ((uint32_t)z << 4));  // 64 + z, ulp 1/16
  return g;
}

// d[i] = (w[i], w[i+4]) dequantized, i = 0..3.
__device__ __forceinline__ void dq_w4(uint32_t w, const W4Group& g, h2 d[4]) {
  const uint32_t w8 = w >> 8;
  // 0x6400 | n reads as 1024 + n; 0x6400 | (n << 4) as 1024 + 16 n.
  const h2 a0 = as_h2((w & 0x000F000Fu) | 0x64006400u);
  const h2 a1 = as_h2((w & 0x00F000F0u) | 0x64006400u);
  const h2 a2 = as_h2((w8 & 0x000F000Fu) | 0x64006400u);
  const h2 a3 = as_h2((w8 & 0x00F000F0u) | 0x64006400u);
  const h2 sixteenth = splat((_Float16)0.0625f);
  d[0] = (a0 - g.zlo) * g.s;                 // (1024 + n) - (1024 + z): exact
  d[1] = (a1 * sixteenth - g.zhi) * g.s;     // (64 + n) - (64 + z): exact
  d[2] = (a2 - g.zlo) * g.s;
  d[3] = (a3 * sixteenth - g.zhi) * g.s;
}

// ---- MXFP4: E2M1 codes with an E8M0 block scale ----------------------------
// A code's magnitude bits i (3 bits) placed at half bits 9..11 read as
// e2m1(i) * 2^-14 (the subnormal encoding covers i = 0, 1), so the element is
// bits * 2^(se - 113).  The power of two is applied as up to three FP16
// multiplies; only the last one that is not 1.0 can round.
struct MxBlock {
  h2 a, b, c;
  bool wide;  // b or c differ from 1.0 (block scale above 2^-98 * 2^113...)
};

__device__ __forceinline__ uint32_t pow2_half_bits(int t) {
  // 2^t for t in [-24, 15] as FP16 bits (subnormal below -14)
  return t >= -14 ? (uint32_t)(t + 15) << 10 : 1u << (t + 24);
}

__device__ __forceinline__ MxBlock mx_block(uint32_t se) {
  const int t = (int)se - 113;
  MxBlock m;
  const int ta = t < -24 ? -24 : (t > 15 ? 15 : t);
  m.a = splat_bits(pow2_half_bits(ta));
  const int tb = t - 15 < 0 ? 0 : (t - 15 > 15 ? 15 : t - 15);
  const int tc = t - 30 < 0 ? 0 : (t - 30 > 15 ? 15 : t - 30);
  m.b = splat_bits(pow2_half_bits(tb));
  m.c = splat_bits(pow2_half_bits(tc));
  m.wide = t > 15;
  return m;
}

// d[i] = (w[i], w[i+4]) dequantized.  `any_wide` is wave-uniform.
__device__ __forceinline__ void dq_mx(uint32_t w, const MxBlock& m, bool any_wide,
                                      h2 d[4]) {
  const uint32_t mag = 0x0E000E00u, sgn = 0x80008000u;
  h2 v0 = as_h2(((w << 9) & mag) | ((w << 12) & sgn));
  h2 v1 = as_h2(((w << 5) & mag) | ((w << 8) & sgn));
  h2 v2 = as_h2(((w << 1) & mag) | ((w << 4) & sgn));
  h2 v3 = as_h2(((w >> 3) & mag) | (w & sgn));
  d[0] = v0 * m.a;
  d[1] = v1 * m.a;
  d[2] = v2 * m.a;
  d[3] = v3 * m.a;
  if (any_wide) {
#pragma unroll
    for (int i = 0; i < 4; ++i) d[i] = (d[i] * m.b) * m.c;
  }
}

// ---- FP8 E4M3 bytes ----------------------------------------------------------
// (b & 0x7F) << 7 read as FP16 is decode(b) * 2^-8 for every code, subnormals
// and the two NaN codes (which the closed-form decode reads as 480) included.
// d[0] = (b0, b2), d[1] = (b1, b3) of the 4-byte word, times the FP16 scale.
__device__ __forceinline__ void dq_f8(uint32_t w, h2 s, h2 d[2]) {
  const h2 k256 = splat((_Float16)256.0f);
  const h2 v0 = as_h2(((w << 7) & 0x3F803F80u) | ((w << 8) & 0x80008000u));
  const h2 v1 = as_h2(((w >> 1) & 0x3F803F80u) | (w & 0x80008000u));
  d[0] = (v0 * k256) * s;
  d[1] = (v1 * k256) * s;
}

// ---- re-pairing ------------------------------------------------------------
// in: d[i] = (e_i, e_{i+4});  out: n[j] = (e_{2j}, e_{2j+1})
__device__ __forceinline__ void to_natural(const h2 d[4], h2 n[4]) {
  n[0] = as_h2(__builtin_amdgcn_perm(as_u32(d[1]), as_u32(d[0]), 0x05040100u));
  n[1] = as_h2(__builtin_amdgcn_perm(as_u32(d[3]), as_u32(d[2]), 0x05040100u));
  n[2] = as_h2(__builtin_amdgcn_perm(as_u32(d[1]), as_u32(d[0]), 0x07060302u));
  n[3] = as_h2(__builtin_amdgcn_perm(as_u32(d[3]), as_u32(d[2]), 0x07060302u));
}

// FP8: d[0] = (e0, e2), d[1] = (e1, e3) -> n[0] = (e0, e1), n[1] = (e2, e3)
__device__ __forceinline__ void to_natural_f8(const h2 d[2], h2 n[2]) {
  n[0] = as_h2(__builtin_amdgcn_perm(as_u32(d[1]), as_u32(d[0]), 0x05040100u));
  n[1] = as_h2(__builtin_amdgcn_perm(as_u32(d[1]), as_u32(d[0]), 0x07060302u));
}

// The same strided pairing applied to 8 activations x0..x7 (16 bytes):
// returns (x0,x4),(x1,x5),(x2,x6),(x3,x7) so dot products line up with dq_*.
__device__ __forceinline__ u4 pair_strided(u4 x) {
  u4 r;
  r[0] = __builtin_amdgcn_perm(x[2], x[0], 0x05040100u);  // x0, x4
  r[1] = __builtin_amdgcn_perm(x[2], x[0], 0x07060302u);  // x1, x5
  r[2] = __builtin_amdgcn_perm(x[3], x[1], 0x05040100u);  // x2, x6
  r[3] = __builtin_amdgcn_perm(x[3], x[1], 0x07060302u);  // x3, x7
  return r;
}

// fp32 accumulate of a packed-half dot: acc + a.x*b.x + a.y*b.y
__device__ __forceinline__ float dot2(h2 a, h2 b, float acc) {
  return __builtin_amdgcn_fdot2(a, b, acc, false);
}

// Wave64 sum of `v`: every lane ends with the total.
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

}  // namespace w4k
