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
// W4 and FP8 pairs come out "strided": register i holds elements (i, i+4) of
// the word (FP8: (i, i+2) of 4 bytes), which is what one mask-and-or per pair
// gives for free.  to_natural() re-pairs them as (0,1),(2,3),(4,5),(6,7) with
// v_perm_b32.  MXFP4 uses the gfx950 FP4 convert and comes out in natural order.
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

// Group index of each of the four 8-k words of a lane's 32-k slice that starts
// at k0 (gs: a multiple of 8).  One division (a shift when gs is a power of two:
// gs_shift >= 0), then compares: 32 k span at most four groups.
// A slice that runs past K (K % 32 != 0) names groups past the last one; they are
// clamped to g_last so that no scale or zero-point is read beyond its row.
__device__ __forceinline__ void groups_of_slice(int k0, int gs, int gs_shift, int g_last,
                                                int g[4]) {
  const int g0 = gs_shift >= 0 ? (k0 >> gs_shift) : k0 / gs;
  const int rem = k0 - g0 * gs;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int o = rem + 8 * j;
    g[j] = min(g0 + (o >= gs) + (o >= 2 * gs) + (o >= 3 * gs), g_last);
  }
}

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

__device__ __forceinline__ W4Group w4_group(_Float16 scale, int z) {
  W4Group g;
  g.s = splat(scale);
  g.zlo = splat_bits(0x6400u | (uint32_t)z);
  g.zhi = splat_bits(0x5400u | ((uint32_t)z << 4));
  return g;
}

// (a & mask) | orv in one VOP3 instruction (the compiler otherwise emits an
// AND and an OR with literal operands).
__device__ __forceinline__ uint32_t and_or(uint32_t a, uint32_t mask, uint32_t orv) {
  uint32_t r;
  asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "s"(mask), "v"(orv));
  return r;
}

// d[i] = (w[i], w[i+4]) dequantized, i = 0..3.
__device__ __forceinline__ void dq_w4(uint32_t w, const W4Group& g, h2 d[4]) {
  const uint32_t w8 = w >> 8;
  uint32_t magic = 0x64006400u;
  asm("" : "+v"(magic));  // keep the constant in a VGPR for the VOP3 form
  // 0x6400 | n reads as 1024 + n; 0x6400 | (n << 4) as 1024 + 16 n.
  const h2 a0 = as_h2(and_or(w, 0x000F000Fu, magic));
  const h2 a1 = as_h2(and_or(w, 0x00F000F0u, magic));
  const h2 a2 = as_h2(and_or(w8, 0x000F000Fu, magic));
  const h2 a3 = as_h2(and_or(w8, 0x00F000F0u, magic));
  const h2 sixteenth = splat((_Float16)0.0625f);
  d[0] = (a0 - g.zlo) * g.s;                 // (1024 + n) - (1024 + z): exact
  d[1] = (a1 * sixteenth - g.zhi) * g.s;     // (64 + n) - (64 + z): exact
  d[2] = (a2 - g.zlo) * g.s;
  d[3] = (a3 * sixteenth - g.zhi) * g.s;
}

// ---- MXFP4: E2M1 codes with an E8M0 block scale ----------------------------
// gfx950 converts two E2M1 codes of one byte, times 2^(exponent of the scale
// operand), to packed FP16 in one instruction.  With the E8M0 byte placed in
// the exponent field of the float operand the result is bit-identical to
// RNE_half(2^(se-127) * e2m1(code)) for every scale byte 0..254 and every code
// (checked exhaustively by the GPU test suite), including results that land in
// the FP16 subnormal range or overflow to infinity.
// n[j] = (w[2j], w[2j+1]): the pairs come out in natural order.
__device__ __forceinline__ float mx_scale(uint32_t se) {
  return __builtin_bit_cast(float, se << 23);
}

__device__ __forceinline__ void dq_mx(uint32_t w, float scale, h2 n[4]) {
  n[0] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, scale, 0);
  n[1] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, scale, 1);
  n[2] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, scale, 2);
  n[3] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, scale, 3);
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

// ---- W4 with the scale and the zero-point outside the inner loop ---------------------
// For results that are not dequantized weights (GEMM outputs of calls without the w_out
// hook):  sum_k x_k s (n_k - z)  =  s * ( sum_k x_k (b_k + n_k)  -  sum_k x_k (b_k + z) ),
// where b_k is the constant that makes a masked nibble an FP16 number with no arithmetic
// at all: 1024 for even k (nibble in the low bits of the significand of 1024.0) and 64
// for odd k (four bits higher, in that of 64.0).  Products of two halves are exact in
// FP32; the biased sum of a 32-k slice stays below 2^17 for activations of unit size,
// so the cancellation costs about 2^-24 * 2^17 against a slice sum of ~ 2^5.
// px: eight activations paired like the codes, (x0,x4),(x1,x5),(x2,x6),(x3,x7).
// ASYM: b += sum_k x_k b_k, a += sum_k x_k over the word (the caller subtracts b + z a).
// Symmetric (z = 8 for every group): b += sum_k x_k (b_k + 8), a is left alone.
template <bool ASYM>
__device__ __forceinline__ void w4_bias_sums(const u4& px, float& b, float& a) {
  const h2 ke = splat((_Float16)(ASYM ? 1024.0f : 1032.0f)), ko = splat((_Float16)(ASYM ? 64.0f : 72.0f));
  b = dot2(as_h2(px[0]), ke, b);
  b = dot2(as_h2(px[1]), ko, b);
  b = dot2(as_h2(px[2]), ke, b);
  b = dot2(as_h2(px[3]), ko, b);
  if (ASYM) {
    const h2 one = splat((_Float16)1.0f);
#pragma unroll
    for (int e = 0; e < 4; ++e) a = dot2(as_h2(px[e]), one, a);
  }
}
// t + sum_k x_k (b_k + n_k) over the word w: a shift, four and-or, four dot products.
__device__ __forceinline__ float w4_dot_biased(uint32_t w, const u4& px, float t) {
  uint32_t m_lo = 0x64006400u, m_hi = 0x54005400u;
  asm("" : "+v"(m_lo), "+v"(m_hi));  // in registers: as literals each and-or becomes two instructions
  const uint32_t w8 = w >> 8;
  t = dot2(as_h2(and_or(w, 0x000F000Fu, m_lo)), as_h2(px[0]), t);   // 1024 + (n0, n4)
  t = dot2(as_h2(and_or(w, 0x00F000F0u, m_hi)), as_h2(px[1]), t);   // 64 + (n1, n5)
  t = dot2(as_h2(and_or(w8, 0x000F000Fu, m_lo)), as_h2(px[2]), t);  // 1024 + (n2, n6)
  t = dot2(as_h2(and_or(w8, 0x00F000F0u, m_hi)), as_h2(px[3]), t);  // 64 + (n3, n7)
  return t;
}
__device__ __forceinline__ float half_bits_to_float(uint32_t b16) {
  return (float)__builtin_bit_cast(_Float16, (uint16_t)b16);
}

// Wave64 sum of `v` with DPP adds only (no LDS traffic): quad swaps, row
// mirrors, then the two row broadcasts.  Lane 63 ends with the total.
template <int CTRL, int ROWMASK>
__device__ __forceinline__ float dpp_add(float v) {
  const int t = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, ROWMASK, 0xF, true);
  return v + __builtin_bit_cast(float, t);
}

__device__ __forceinline__ float wave_sum_to_lane63(float v) {
  v = dpp_add<0xB1, 0xF>(v);   // quad_perm [1,0,3,2]
  v = dpp_add<0x4E, 0xF>(v);   // quad_perm [2,3,0,1]
  v = dpp_add<0x141, 0xF>(v);  // row_half_mirror
  v = dpp_add<0x140, 0xF>(v);  // row_mirror: every lane of a row holds the row sum
  v = dpp_add<0x142, 0xA>(v);  // row_bcast15 into rows 1 and 3
  v = dpp_add<0x143, 0xC>(v);  // row_bcast31 into rows 2 and 3
  return v;
}

}  // namespace w4k
