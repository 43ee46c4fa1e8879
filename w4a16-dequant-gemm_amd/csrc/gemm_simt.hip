// Fused dequant + GEMM on the vector ALUs: c[m,n] = sum_k x[m,k] * W[n,k] with
// W streamed once from HBM as packed 4-bit codes and expanded in VGPRs.
//
// Mapping (wave64): a wave owns R weight rows; per 2048-k block each lane
// fetches one dwordx4 of each row (4 packed words = 32 consecutive k; 1 KiB per
// row per wave, fully coalesced) and the matching 32 activations of each of
// the MT activation rows from LDS.  Products are v_dot2_f32_f16 into FP32
// accumulators; the K reduction is finished with DPP adds.
//
// Memory returns loads in issue order, so the order of requests is part of the
// design: the activations first (the staging barrier then waits for nothing
// else), block 0 of the weights right behind them (in flight across the
// barrier), and block b+1 (codes, scales, zero-points) before block b is
// expanded, so HBM latency overlaps the barrier and the ALU work.
//
// Activations are staged in LDS once per workgroup, paired to match what the
// dequant step produces ((k, k+4) for W4, natural for MXFP4), and laid out so
// that lane l reads 16-byte slot (j*64 + l): consecutive lanes, consecutive
// banks.
//
// The fast kernel needs 16-byte-aligned rows (K % 32 == 0, aligned bases).
// Otherwise lanes walk single words (ragged K, K = 4104, 72, 100 ...).
#include <utility>

#include "dq.cuh"
#include "kernels.h"
#include "simt_rows4.cuh"

namespace w4k {

constexpr int SIMT_R = 2;               // weight rows per wave
constexpr int KS_R = 4;                 // weight rows per workgroup of the K-split kernel
constexpr int SIMT_LDS_HALVES = 16384;  // activations resident in LDS at once (32 KiB)

__device__ __forceinline__ u4 load_x8_guarded(const w4_half* __restrict__ x, int M, int K,
                                              int row, int k, bool x_vec) {
  u4 v = {0u, 0u, 0u, 0u};
  if (row < M && k < K) {
    const uint16_t* src = x + (size_t)row * K + k;
    if (x_vec && k + 8 <= K) {
      v = *(const u4*)src;
    } else {
      uint16_t t[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) t[j] = (k + j < K) ? src[j] : (uint16_t)0;
      v = u4{t[0] | ((uint32_t)t[1] << 16), t[2] | ((uint32_t)t[3] << 16),
             t[4] | ((uint32_t)t[5] << 16), t[6] | ((uint32_t)t[7] << 16)};
    }
  }
  return v;
}

// Stage x[m0 .. m0+MT)[kc .. kc+kc_len) into LDS, zero-filled past M and K.
// SLOTTED: the slot of 8-group g8 is (g8 & ~255) + (g8 & 3) * 64 + ((g8 & 255) >> 2).
template <int MX, int MT, bool SLOTTED>
__device__ __forceinline__ void stage_x(u4* xs, const w4_half* __restrict__ x, int M,
                                        int K, int m0, int kc, int groups, int slots,
                                        bool x_vec) {
  for (int i = threadIdx.x; i < slots * MT; i += SIMT_WAVES * 64) {
    const int m = i / slots, g8 = i - m * slots;
    u4 v = {0u, 0u, 0u, 0u};
    if (g8 < groups) v = load_x8_guarded(x, M, K, m0 + m, kc + g8 * 8, x_vec);
    const int slot = SLOTTED ? (g8 & ~255) + (g8 & 3) * 64 + ((g8 & 255) >> 2) : g8;
    xs[m * slots + slot] = MX ? v : pair_strided(v);
  }
}

__device__ __forceinline__ int zero_point(const WView& p, int n, int g, int wg) {
  return p.symmetric ? 8 : (int)((p.zeros[(size_t)n * wg + (g >> 3)] >> (4 * (g & 7))) & 0xF);
}

// One block of one lane: R rows x 4 words, plus the group parameters they need.
template <int MX, int R, bool GS32>
struct LaneBlock {
  static constexpr int NS = (MX || GS32) ? 1 : 4;
  u4 q[R];
  uint32_t s[R][NS];  // scale bits (FP16) or E8M0 byte
  uint32_t z[R][NS];  // zero-point (W4)
};

template <int MX, int R, bool GS32>
__device__ __forceinline__ void load_block(LaneBlock<MX, R, GS32>& b, const WView& p, int n0,
                                           int wpr, int wg, int w0) {
  constexpr int NS = LaneBlock<MX, R, GS32>::NS;
  const bool active = w0 < wpr;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int n = min(n0 + r, p.N - 1);
    b.q[r] = u4{0u, 0u, 0u, 0u};
#pragma unroll
    for (int i = 0; i < NS; ++i) b.s[r][i] = 0u, b.z[r][i] = 8u;
    if (active) {
      b.q[r] = __builtin_nontemporal_load((const u4*)(p.q + (size_t)n * wpr + w0));
      if (MX) {
        b.s[r][0] = ((const uint8_t*)p.scales)[(size_t)n * p.B + (w0 >> 2)];
      } else {
#pragma unroll
        for (int i = 0; i < NS; ++i) {
          const int g = (8 * (w0 + i)) / p.gs;
          b.s[r][i] = ((const uint16_t*)p.scales)[(size_t)n * p.G + g];
          b.z[r][i] = (uint32_t)zero_point(p, n, g, wg);
        }
      }
    }
  }
}

template <int MX, int MT, int R, bool HOOK, bool GS32>
__global__ __launch_bounds__(SIMT_WAVES * 64) void simt_fast_kernel(
    const WView p, const w4_half* __restrict__ x, w4_half* __restrict__ c, const int M,
    w4_half* __restrict__ w_out, const bool x_vec) {
  extern __shared__ u4 xs[];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n0 = (blockIdx.x * SIMT_WAVES + wave) * R;
  const int m0 = blockIdx.y * MT;
  const int wpr = words(p.K);
  const bool hook = HOOK && blockIdx.y == 0;
  const int wg = MX ? 0 : words(p.G);
  const bool wave_on = n0 < p.N;  // wave-uniform
  constexpr int KC = SIMT_LDS_HALVES / MT;  // k range staged per pass (multiple of 2048)
  constexpr int NS = LaneBlock<MX, R, GS32>::NS;

  float acc[R][MT];
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int m = 0; m < MT; ++m) acc[r][m] = 0.0f;

  LaneBlock<MX, R, GS32> cur, nxt;

  const int nblk = (wpr + 255) / 256;
  for (int kc = 0, blk0 = 0; kc < p.K; kc += KC, blk0 += KC / 2048) {
    const int kc_len = min(KC, p.K - kc);
    const int groups = kc_len >> 3;  // K % 32 == 0 here
    const int slots = (groups + 255) & ~255;
    if (kc) __syncthreads();
    // Loads return in issue order: the activations are requested first so the
    // staging barrier only waits for them, and the first weight block is
    // requested right behind them so it is in flight across the barrier.
    constexpr int XL = (KC / 8 * MT + SIMT_WAVES * 64 - 1) / (SIMT_WAVES * 64);
    u4 xv[XL];
#pragma unroll
    for (int t = 0; t < XL; ++t) {
      const int i = t * SIMT_WAVES * 64 + threadIdx.x;
      const int m = i / slots, g8 = i - m * slots;
      xv[t] = u4{0u, 0u, 0u, 0u};
      if (i < slots * MT && g8 < groups) xv[t] = load_x8_guarded(x, M, p.K, m0 + m, kc + g8 * 8, x_vec);
    }
    if (kc == 0 && wave_on) load_block(cur, p, n0, wpr, wg, lane * 4);
#pragma unroll
    for (int t = 0; t < XL; ++t) {
      const int i = t * SIMT_WAVES * 64 + threadIdx.x;
      const int m = i / slots, g8 = i - m * slots;
      const int slot = (g8 & ~255) + (g8 & 3) * 64 + ((g8 & 255) >> 2);
      if (i < slots * MT) xs[m * slots + slot] = MX ? xv[t] : pair_strided(xv[t]);
    }
    __syncthreads();
    if (!wave_on) continue;

    const int blk1 = min(nblk, blk0 + KC / 2048);
    for (int blk = blk0; blk < blk1; ++blk) {
      if (blk + 1 < nblk) load_block(nxt, p, n0, wpr, wg, (blk + 1) * 256 + lane * 4);
      const int lb = blk - blk0;
      u4 xr[MT][4];
#pragma unroll
      for (int m = 0; m < MT; ++m)
#pragma unroll
        for (int j = 0; j < 4; ++j) xr[m][j] = xs[m * slots + lb * 256 + j * 64 + lane];
      const int k0 = (blk * 256 + lane * 4) * 8;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const int n = min(n0 + r, p.N - 1);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          h2 d[4];
          if (MX) {
            dq_mx(cur.q[r][j], mx_scale(cur.s[r][0]), d);
          } else {
            const int i = NS == 1 ? 0 : j;
            dq_w4(cur.q[r][j], w4_group((uint16_t)cur.s[r][i], (int)cur.z[r][i]), d);
          }
#pragma unroll
          for (int m = 0; m < MT; ++m)
#pragma unroll
            for (int e = 0; e < 4; ++e)
              acc[r][m] = dot2(d[e], as_h2(xr[m][j][e]), acc[r][m]);
          if (hook && n0 + r < p.N && k0 < p.K) {
            h2 nat[4];
            if (MX) {
#pragma unroll
              for (int e = 0; e < 4; ++e) nat[e] = d[e];
            } else {
              to_natural(d, nat);
            }
            *(u4*)(w_out + (size_t)n * p.K + k0 + 8 * j) =
                u4{as_u32(nat[0]), as_u32(nat[1]), as_u32(nat[2]), as_u32(nat[3])};
          }
        }
      }
      if (blk + 1 < nblk) cur = nxt;
    }
  }

  if (!wave_on) return;
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int m = 0; m < MT; ++m) acc[r][m] = wave_sum_to_lane63(acc[r][m]);
  if (lane == 63) {
    const bool pair_ok = R == 2 && (p.N & 1) == 0 && (((uintptr_t)c & 3) == 0) && n0 + 1 < p.N;
#pragma unroll
    for (int m = 0; m < MT; ++m) {
      if (m0 + m >= M) continue;
      uint16_t* dst = c + (size_t)(m0 + m) * p.N + n0;
      if (pair_ok) {  // the wave's two rows leave as one 4-byte store
        const _Float16 h0 = (_Float16)acc[0][m], h1 = (_Float16)acc[R - 1][m];
        *(uint32_t*)dst = (uint32_t)__builtin_bit_cast(uint16_t, h0) |
                          ((uint32_t)__builtin_bit_cast(uint16_t, h1) << 16);
      } else {
#pragma unroll
        for (int r = 0; r < R; ++r)
          if (n0 + r < p.N) {
            const _Float16 h = (_Float16)acc[r][m];
            dst[r] = __builtin_bit_cast(uint16_t, h);
          }
      }
    }
  }
}

// Any K, any alignment: one packed word per lane per step.
template <int MX, int MT, int R, bool HOOK>
__global__ __launch_bounds__(SIMT_WAVES * 64) void simt_generic_kernel(
    const WView p, const w4_half* __restrict__ x, w4_half* __restrict__ c, const int M,
    w4_half* __restrict__ w_out, const bool x_vec) {
  extern __shared__ u4 xs[];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n0 = (blockIdx.x * SIMT_WAVES + wave) * R;
  const int m0 = blockIdx.y * MT;
  const int wpr = words(p.K);
  const bool hook = HOOK && blockIdx.y == 0;
  const int wg = MX ? 0 : words(p.G);
  const bool wave_on = n0 < p.N;
  constexpr int KC = SIMT_LDS_HALVES / MT;

  float acc[R][MT];
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int m = 0; m < MT; ++m) acc[r][m] = 0.0f;

  for (int kc = 0; kc < p.K; kc += KC) {
    const int kc_len = min(KC, p.K - kc);
    const int groups = (kc_len + 7) >> 3;
    if (kc) __syncthreads();
    stage_x<MX, MT, false>(xs, x, M, p.K, m0, kc, groups, groups, x_vec);
    __syncthreads();
    if (!wave_on) continue;
    for (int wi = lane; wi < groups; wi += 64) {
      const int k0 = kc + wi * 8;
      u4 xr[MT];
#pragma unroll
      for (int m = 0; m < MT; ++m) xr[m] = xs[m * groups + wi];
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const int n = min(n0 + r, p.N - 1);
        const uint32_t qw = p.q[(size_t)n * wpr + (k0 >> 3)];
        h2 d[4];
        if (MX) {
          dq_mx(qw, mx_scale(((const uint8_t*)p.scales)[(size_t)n * p.B + (k0 >> 5)]), d);
        } else {
          const int g = k0 / p.gs;
          dq_w4(qw, w4_group(((const uint16_t*)p.scales)[(size_t)n * p.G + g],
                             zero_point(p, n, g, wg)), d);
        }
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
          for (int e = 0; e < 4; ++e) acc[r][m] = dot2(d[e], as_h2(xr[m][e]), acc[r][m]);
        if (hook && n0 + r < p.N) {
          h2 nat[4];
          if (MX) {
#pragma unroll
            for (int e = 0; e < 4; ++e) nat[e] = d[e];
          } else {
            to_natural(d, nat);
          }
          uint16_t* out = w_out + (size_t)n * p.K + k0;
#pragma unroll
          for (int j = 0; j < 8; ++j)
            if (k0 + j < p.K) {
              const uint32_t pair = as_u32(nat[j >> 1]);
              out[j] = (uint16_t)((j & 1) ? pair >> 16 : pair & 0xFFFFu);
            }
        }
      }
    }
  }

  if (!wave_on) return;
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int m = 0; m < MT; ++m) acc[r][m] = wave_sum_to_lane63(acc[r][m]);
  if (lane == 63) {
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int m = 0; m < MT; ++m)
        if (n0 + r < p.N && m0 + m < M) {
          const _Float16 h = (_Float16)acc[r][m];
          c[(size_t)(m0 + m) * p.N + n0 + r] = __builtin_bit_cast(uint16_t, h);
        }
  }
}

// Fully unrolled form of the fast kernel for the shapes decode GEMMs have:
// K = STEPS * 2048, one group per 32-k lane slice, whole workgroups of rows, no
// hook.  Every load of a wave (activations first, then the scales, then the
// STEPS * R weight dwordx4) is issued before anything is consumed, and the
// waits are retired in that order.
template <int MX, int MT, int R, int STEPS, bool ASYM, bool POW2, bool GS32>
__global__ __launch_bounds__(SIMT_WAVES * 64) void simt_unrolled_kernel(
    const WView p, const w4_half* __restrict__ x, w4_half* __restrict__ c, const int M,
    const int gs_shift) {
  // One activation row: every lane fetches its own 32-k slices of x straight from
  // L2 (no LDS, no barrier: 0.3 us at N = K = 4096).  More rows: staged once per
  // workgroup in LDS.
  constexpr bool XDIRECT = MT == 1;
  __shared__ u4 xs[XDIRECT ? 1 : MT * STEPS * 256];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n0 = (blockIdx.x * SIMT_WAVES + wave) * R;
  const int m0 = blockIdx.y * MT;
  constexpr int K = STEPS * 2048, WPR = K / 8;
  constexpr int XL = XDIRECT ? STEPS * 4 : (MT * STEPS * 256) / (SIMT_WAVES * 64);
  const int wg = MX ? 0 : words(p.G);

  const u4* xsrc[XL];
#pragma unroll
  for (int t = 0; t < XL; ++t) {
    if (XDIRECT) {
      xsrc[t] = (const u4*)(x + (size_t)m0 * K + (t >> 2) * 2048 + lane * 32 + (t & 3) * 8);
    } else {
      const int i = t * SIMT_WAVES * 64 + threadIdx.x;
      const int m = min(i / (STEPS * 256), M - 1 - m0), g8 = i % (STEPS * 256);
      xsrc[t] = (const u4*)(x + (size_t)(m0 + m) * K + g8 * 8);  // rows past M: a valid row, never stored
    }
  }
  constexpr int NS = (MX || GS32) ? 1 : 4;  // group lookups per lane slice
  const uint16_t* ssrc[STEPS][R][NS];
  const uint32_t* zsrc[STEPS][R][NS];
  uint32_t zsh[STEPS][NS];
  const u4* qsrc[STEPS][R];
#pragma unroll
  for (int s = 0; s < STEPS; ++s) {
    const int k0 = s * 2048 + lane * 32;
    int g[4];
    if (NS == 1) g[0] = MX ? (k0 >> 5) : POW2 ? (k0 >> gs_shift) : k0 / p.gs;
    else groups_of_slice(k0, p.gs, gs_shift, p.G - 1, g);
#pragma unroll
    for (int e = 0; e < NS; ++e) zsh[s][e] = 4u * (uint32_t)(g[e] & 7);
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const size_t n = (size_t)(n0 + r);
#pragma unroll
      for (int e = 0; e < NS; ++e) {
        ssrc[s][r][e] = MX ? (const uint16_t*)((const uint8_t*)p.scales + n * p.B + g[e])
                           : (const uint16_t*)p.scales + n * p.G + g[e];
        zsrc[s][r][e] = ASYM ? p.zeros + n * wg + (g[e] >> 3) : nullptr;
      }
      qsrc[s][r] = (const u4*)(p.q + n * WPR + s * 256 + lane * 4);
    }
  }
  u4 xv[XL];
  uint32_t sc[STEPS][R][NS], zw[STEPS][R][NS];
  u4 qw[STEPS][R];
#pragma unroll
  for (int t = 0; t < XL; ++t) xv[t] = *xsrc[t];
#pragma unroll
  for (int s = 0; s < STEPS; ++s)
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int e = 0; e < NS; ++e) {
        sc[s][r][e] = MX ? (uint32_t) * (const uint8_t*)ssrc[s][r][e] : (uint32_t)*ssrc[s][r][e];
        zw[s][r][e] = ASYM ? *zsrc[s][r][e] : 0u;
      }
#pragma unroll
  for (int s = 0; s < STEPS; ++s)
#pragma unroll
    for (int r = 0; r < R; ++r) qw[s][r] = __builtin_nontemporal_load(qsrc[s][r]);
  // With LDS staging every request goes out before the barrier.  With direct
  // activations the compiler is left free to weave address arithmetic between
  // the requests and to start on the first rows while the last request is still
  // being formed: measured 3.8 us against 4.2 us with all requests forced up
  // front (N = K = 4096) -- at kernel start the 16 waves of a CU all compete for
  // the vector ALUs, so what matters is how few instructions precede each request.
  if (!XDIRECT) __builtin_amdgcn_sched_barrier(0);
  if (!XDIRECT) {
#pragma unroll
    for (int t = 0; t < XL; ++t) {
      const int i = t * SIMT_WAVES * 64 + threadIdx.x;
      const int m = i / (STEPS * 256), g8 = i % (STEPS * 256);
      const int slot = (g8 & ~255) + (g8 & 3) * 64 + ((g8 & 255) >> 2);
      xs[m * STEPS * 256 + slot] = MX ? xv[t] : pair_strided(xv[t]);
    }
    __syncthreads();
  }

  float acc[R][MT];
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int m = 0; m < MT; ++m) acc[r][m] = 0.0f;
#pragma unroll
  for (int s = 0; s < STEPS; ++s) {
    u4 xr[MT][4];
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (XDIRECT) xr[m][j] = MX ? xv[s * 4 + j] : pair_strided(xv[s * 4 + j]);
        else xr[m][j] = xs[m * STEPS * 256 + s * 256 + j * 64 + lane];
      }
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const float mxs = mx_scale(sc[s][r][0]);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int e = NS == 1 ? 0 : j;
        h2 d[4];
        if (MX)
          dq_mx(qw[s][r][j], mxs, d);
        else
          dq_w4(qw[s][r][j],
                w4_group((uint16_t)sc[s][r][e], ASYM ? (int)((zw[s][r][e] >> zsh[s][e]) & 0xFu) : 8), d);
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
          for (int e = 0; e < 4; ++e) acc[r][m] = dot2(d[e], as_h2(xr[m][j][e]), acc[r][m]);
      }
    }
  }
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int m = 0; m < MT; ++m) acc[r][m] = wave_sum_to_lane63(acc[r][m]);
  if (lane == 63) {
#pragma unroll
    for (int m = 0; m < MT; ++m) {
      if (m0 + m >= M) continue;
      uint16_t* dst = c + (size_t)(m0 + m) * p.N + n0;
      if (R == 2) {  // N is a multiple of 8 here, so the pair is 4-byte aligned with c
        const _Float16 h0 = (_Float16)acc[0][m], h1 = (_Float16)acc[R - 1][m];
        *(uint32_t*)dst = (uint32_t)__builtin_bit_cast(uint16_t, h0) |
                          ((uint32_t)__builtin_bit_cast(uint16_t, h1) << 16);
      } else {
#pragma unroll
        for (int r = 0; r < R; ++r) {
          const _Float16 h = (_Float16)acc[r][m];
          dst[r] = __builtin_bit_cast(uint16_t, h);
        }
      }
    }
  }
}

template <int MX, int MT, int STEPS>
static hipError_t launch_rows4(const WView& v, const w4_half* x, w4_half* c, int M, hipStream_t s) {
  const dim3 grid((unsigned)(v.N / (SIMT_WAVES * ROWS4_R)), (unsigned)((M + MT - 1) / MT));
  // a power of two 32 .. 256: its shift; any other gs % 8 == 0: 0 (gs >= 32) or 3 (gs >= 8)
  const bool pow2 = MX || (v.gs & (v.gs - 1)) == 0;
  const int gsh = MX ? 5 : pow2 && v.gs >= 32 && v.gs <= 256 ? __builtin_ctz((unsigned)v.gs) : v.gs >= 32 ? 0 : 3;
#define W4_GO(ASYM, GSH)                                                               \
  simt_rows4_kernel<MX, MT, STEPS, ASYM, GSH, false><<<grid, SIMT_WAVES * 64, 0, s>>>( \
      v.q, v.scales, v.zeros, x, c, v.N, M, v.gs, v.G, nullptr)
  // (a group lookup per packed word with eight activation rows needs more registers than
  // a lane has: try_rows4 leaves those calls to the kernels below)
#define W4_GSH(ASYM)                                                          \
  switch (gsh) {                                                              \
    case 0: if constexpr (MT <= 4) W4_GO(ASYM, 0); break;                     \
    case 3: if constexpr (MT <= 4) W4_GO(ASYM, 3); break;                     \
    case 5: W4_GO(ASYM, 5); break;                                            \
    case 6: W4_GO(ASYM, 6); break;                                            \
    case 7: W4_GO(ASYM, 7); break;                                            \
    default: W4_GO(ASYM, 8); break;                                           \
  }
  if constexpr (MX) W4_GO(false, 5);
  else if (v.symmetric) { W4_GSH(false) }
  else { W4_GSH(true) }
#undef W4_GSH
#undef W4_GO
  return hipGetLastError();
}

// true (and launched) when the four-rows-per-wave kernel applies
template <int MX, int MT>
static bool try_rows4(const WView& v, const w4_half* x, w4_half* c, int M, hipStream_t s,
                      w4_half* w_out, hipError_t* err) {
  if (w_out || v.K % 2048 || v.N % (SIMT_WAVES * ROWS4_R)) return false;
  if (!MX && (v.gs < 8 || v.gs % 8)) return false;
  const bool one_group_per_slice = MX || ((v.gs & (v.gs - 1)) == 0 && v.gs >= 32 && v.gs <= 256);
  if (MT > 4 && !one_group_per_slice) return false;
  if ((((uintptr_t)v.q | (uintptr_t)x) & 15) || ((uintptr_t)c & 7) || ((uintptr_t)v.scales & 3))
    return false;
  const int steps = v.K / 2048;
  if (steps * MT > 8) return false;  // LDS: MT * K halves, at most 32 KiB
  switch (steps) {
    case 1: *err = launch_rows4<MX, MT, 1>(v, x, c, M, s); return true;
    case 2: if constexpr (MT <= 4) { *err = launch_rows4<MX, MT <= 4 ? MT : 1, 2>(v, x, c, M, s); return true; } return false;
    case 4: if constexpr (MT <= 2) { *err = launch_rows4<MX, MT <= 2 ? MT : 1, 4>(v, x, c, M, s); return true; } return false;
    default: return false;
  }
}

// One or two activation rows, long or odd K (K % 32 == 0, K <= 16384; e.g. 11008,
// 14336, 6144): the W waves of a workgroup share R = 4 weight rows (a wave's slice of
// the activations serves all of them: two rows per workgroup read the activations
// from L2 twice as often and took 8.4 instead of 7.0 us at N = 4096, K = 11008; eight
// rows leave too few workgroups) and split K into
// runs of whole 32-k slices (W is chosen so that the lanes are nearly all busy:
// 6 waves for K = 11008, 7 for 14336); each wave is the unrolled kernel on its run
// (activations straight from L2, everything requested before it is consumed,
// lanes past the end of the quarter clamped to k = 0 with zeroed activations),
// and the partial sums meet in LDS in wave order.
template <int MX, int MT, int R, int W, int STEPS, bool ASYM, bool GS32, bool HOOK>
__global__ __launch_bounds__(W * 64) void simt_ksplit_kernel(
    const uint32_t* __restrict__ q_, const void* __restrict__ scales_,
    const w4_half* __restrict__ x, w4_half* __restrict__ c, const int K_, const int N_,
    const int M, const int gs_shift, const int G_, const int gs_,
    const uint32_t* __restrict__ zeros_, w4_half* __restrict__ w_out) {
  // the leading arguments arrive in registers with the wave: the code stream is addressed
  // without a round trip to the argument segment
  const struct { const uint32_t* q; const void* scales; const uint32_t* zeros; int K, N, G, B, gs; }
      p{q_, scales_, zeros_, K_, N_, G_, G_, gs_};
  __shared__ float red[W][R][MT];
  constexpr int NS = (MX || GS32) ? 1 : 4;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n0 = blockIdx.x * R;
  const int m0 = blockIdx.y * MT;
  const int wpr = p.K >> 3;
  const int wg = MX ? 0 : words(p.G);
  const int slices = p.K >> 5;                              // 32-k slices in a row
  const int per = (slices + W - 1) / W;                     // ... per wave
  const int s_lo = wave * per, s_hi = min(slices, s_lo + per);
  const bool hook = HOOK && blockIdx.y == 0;

  int k0[STEPS];
  bool on[STEPS];
#pragma unroll
  for (int s = 0; s < STEPS; ++s) {
    const int sl = s_lo + s * 64 + lane;
    on[s] = sl < s_hi;
    k0[s] = on[s] ? sl * 32 : 0;
  }
  u4 xv[STEPS][MT][4];
#pragma unroll
  for (int s = 0; s < STEPS; ++s)
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
      for (int j = 0; j < 4; ++j)  // rows past M repeat the last row and are never stored
        xv[s][m][j] = *(const u4*)(x + (size_t)min(m0 + m, M - 1) * p.K + k0[s] + 8 * j);
  uint32_t sc[STEPS][R][NS], zw[STEPS][R][NS], zsh[STEPS][NS];
#pragma unroll
  for (int s = 0; s < STEPS; ++s) {
    int g[4];
    if (NS == 1) g[0] = MX ? (k0[s] >> 5) : gs_shift >= 0 ? (k0[s] >> gs_shift) : k0[s] / p.gs;
    else groups_of_slice(k0[s], p.gs, gs_shift, p.G - 1, g);
#pragma unroll
    for (int e = 0; e < NS; ++e) {
      zsh[s][e] = 4u * (uint32_t)(g[e] & 7);
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const size_t n = (size_t)(n0 + r);
        sc[s][r][e] = MX ? (uint32_t)((const uint8_t*)p.scales)[n * p.B + g[e]]
                         : (uint32_t)((const uint16_t*)p.scales)[n * p.G + g[e]];
        zw[s][r][e] = ASYM ? p.zeros[n * wg + (g[e] >> 3)] : 0u;
      }
    }
  }
  u4 qw[STEPS][R];
#pragma unroll
  for (int s = 0; s < STEPS; ++s)
#pragma unroll
    for (int r = 0; r < R; ++r) {
      qw[s][r] = __builtin_nontemporal_load((const u4*)(p.q + (size_t)(n0 + r) * wpr + (k0[s] >> 3)));
    }

  float acc[R][MT];
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int m = 0; m < MT; ++m) acc[r][m] = 0.0f;
#pragma unroll
  for (int s = 0; s < STEPS; ++s) {
    u4 xr[MT][4];
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        xr[m][j] = MX ? xv[s][m][j] : pair_strided(xv[s][m][j]);
        if (!on[s]) xr[m][j] = u4{0u, 0u, 0u, 0u};
      }
    if constexpr (!MX && !HOOK) {
      // no dequantized weight leaves this instantiation: biased codes, the scale and the
      // zero-point applied once per group in FP32 (w4_dot_biased); the bias sums of the
      // lane's slice serve all R rows
      float pb[MT][NS], pa[MT][NS];
#pragma unroll
      for (int m = 0; m < MT; ++m) {
#pragma unroll
        for (int e = 0; e < NS; ++e) pb[m][e] = pa[m][e] = 0.0f;
#pragma unroll
        for (int j = 0; j < 4; ++j) w4_bias_sums<ASYM>(xr[m][j], pb[m][NS == 1 ? 0 : j], pa[m][NS == 1 ? 0 : j]);
      }
#pragma unroll
      for (int r = 0; r < R; ++r) {
        float t[MT];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int e = NS == 1 ? 0 : j;
          if (NS == 4 || j == 0) {
            const float z = (float)((zw[s][r][e] >> zsh[s][e]) & 0xFu);
#pragma unroll
            for (int m = 0; m < MT; ++m) t[m] = ASYM ? -__builtin_fmaf(z, pa[m][e], pb[m][e]) : -pb[m][e];
          }
#pragma unroll
          for (int m = 0; m < MT; ++m) t[m] = w4_dot_biased(qw[s][r][j], xr[m][j], t[m]);
          if (NS == 4 || j == 3) {
            const float sf = half_bits_to_float(sc[s][r][e]);
#pragma unroll
            for (int m = 0; m < MT; ++m) acc[r][m] = __builtin_fmaf(sf, t[m], acc[r][m]);
          }
        }
      }
      continue;
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const float mxs = mx_scale(sc[s][r][0]);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int e = NS == 1 ? 0 : j;
        h2 d[4];
        if (MX)
          dq_mx(qw[s][r][j], mxs, d);
        else
          dq_w4(qw[s][r][j],
                w4_group((uint16_t)sc[s][r][e], ASYM ? (int)((zw[s][r][e] >> zsh[s][e]) & 0xFu) : 8), d);
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
          for (int t = 0; t < 4; ++t) acc[r][m] = dot2(d[t], as_h2(xr[m][j][t]), acc[r][m]);
        if (hook && on[s]) {
          h2 nat[4];
          if (MX) {
#pragma unroll
            for (int t = 0; t < 4; ++t) nat[t] = d[t];
          } else {
            to_natural(d, nat);
          }
          *(u4*)(w_out + (size_t)(n0 + r) * p.K + k0[s] + 8 * j) =
              u4{as_u32(nat[0]), as_u32(nat[1]), as_u32(nat[2]), as_u32(nat[3])};
        }
      }
    }
  }
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int m = 0; m < MT; ++m) acc[r][m] = wave_sum_to_lane63(acc[r][m]);
  if (lane == 63) {
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int m = 0; m < MT; ++m) red[wave][r][m] = acc[r][m];
  }
  __syncthreads();
  if (threadIdx.x < R * MT) {
    const int r = threadIdx.x / MT, m = threadIdx.x % MT;
    float sum = red[0][r][m];
#pragma unroll
    for (int w = 1; w < W; ++w) sum += red[w][r][m];
    if (m0 + m < M) {
      const _Float16 h = (_Float16)sum;
      c[(size_t)(m0 + m) * p.N + n0 + r] = __builtin_bit_cast(uint16_t, h);
    }
  }
}

template <int MX, int MT, int W, int STEPS>
static hipError_t launch_ksplit(const WView& v, const w4_half* x, w4_half* c, int M, hipStream_t s,
                                w4_half* w_out) {
  const bool gs32 = MX || v.gs % 32 == 0;
  const bool pow2 = !MX && (v.gs & (v.gs - 1)) == 0;
  const int sh = pow2 ? __builtin_ctz((unsigned)v.gs) : -1;
  const dim3 grid((unsigned)(v.N / KS_R), (unsigned)((M + MT - 1) / MT));
#define W4_GO(ASYM, GS32)                                                                 \
  do {                                                                                    \
    if (w_out)                                                                            \
      simt_ksplit_kernel<MX, MT, KS_R, W, STEPS, ASYM, GS32, true>                      \
          <<<grid, W * 64, 0, s>>>(v.q, v.scales, x, c, v.K, v.N, M, sh, MX ? v.B : v.G,  \
                                   v.gs, v.zeros, w_out);                                 \
    else                                                                                  \
      simt_ksplit_kernel<MX, MT, KS_R, W, STEPS, ASYM, GS32, false>                     \
          <<<grid, W * 64, 0, s>>>(v.q, v.scales, x, c, v.K, v.N, M, sh, MX ? v.B : v.G,  \
                                   v.gs, v.zeros, w_out);                                 \
  } while (0)
  if (!MX && !v.symmetric) {
    if (gs32) W4_GO(true, true); else W4_GO(true, false);
  } else {
    if (gs32) W4_GO(false, true); else W4_GO(false, false);
  }
#undef W4_GO
  return hipGetLastError();
}

template <int MX, int MT>
static bool try_ksplit(const WView& v, const w4_half* x, w4_half* c, int M, hipStream_t s,
                       w4_half* w_out, hipError_t* err) {
  // four rows fetched per wave cost more than the staged kernel's barrier (20.7 vs 19 us at K = 11008)
  if (MT > 2 || v.K % 32 || v.K > 16384 || v.K < 2048 || v.N % KS_R) return false;
  // shapes of the unrolled kernel stay with it (and, hooked, with the kernel that sums like it)
  const int blocks = v.K / 2048;
  if (v.K % 2048 == 0 && (blocks == 1 || blocks == 2 || blocks == 4) && blocks * MT <= 8 &&
      v.N % (SIMT_WAVES * SIMT_R) == 0)
    return false;
  if ((((uintptr_t)v.q | (uintptr_t)x | (uintptr_t)w_out) & 15)) return false;
  const int slices = v.K >> 5;  // 64 ... 512
  // fewest waves (at least 4) that cover the row in one step of 64 slices each; two steps past 512
  if (slices <= 256) *err = launch_ksplit<MX, MT <= 2 ? MT : 1, 4, 1>(v, x, c, M, s, w_out);
  else if (slices <= 320) *err = launch_ksplit<MX, MT <= 2 ? MT : 1, 5, 1>(v, x, c, M, s, w_out);
  else if (slices <= 384) *err = launch_ksplit<MX, MT <= 2 ? MT : 1, 6, 1>(v, x, c, M, s, w_out);
  else if (slices <= 448) *err = launch_ksplit<MX, MT <= 2 ? MT : 1, 7, 1>(v, x, c, M, s, w_out);
  else *err = launch_ksplit<MX, MT <= 2 ? MT : 1, 8, 1>(v, x, c, M, s, w_out);
  return true;
}

template <int MX, int MT, int STEPS>
static hipError_t launch_unrolled(const WView& v, const w4_half* x, w4_half* c, int M,
                                  hipStream_t s) {
  const dim3 grid((unsigned)(v.N / (SIMT_WAVES * SIMT_R)), (unsigned)((M + MT - 1) / MT));
  const bool pow2 = !MX && (v.gs & (v.gs - 1)) == 0;  // group index by shift instead of division
  const int sh = pow2 ? __builtin_ctz((unsigned)v.gs) : 0;
  const bool gs32 = MX || v.gs % 32 == 0;  // else a lane's 32-k slice spans several groups
#define W4_GO(ASYM, POW2, GS32) \
  simt_unrolled_kernel<MX, MT, SIMT_R, STEPS, ASYM, POW2, GS32> \
      <<<grid, SIMT_WAVES * 64, 0, s>>>(v, x, c, M, pow2 ? sh : -1)
  if (!gs32) {
    if (!v.symmetric) W4_GO(true, false, false); else W4_GO(false, false, false);
  } else if (!MX && !v.symmetric) {
    if (pow2) W4_GO(true, true, true); else W4_GO(true, false, true);
  } else {
    if (pow2) W4_GO(false, true, true); else W4_GO(false, false, true);
  }
#undef W4_GO
  return hipGetLastError();
}

// true (and launched) when the unrolled kernel applies
template <int MX, int MT>
static bool try_unrolled(const WView& v, const w4_half* x, w4_half* c, int M, hipStream_t s,
                         w4_half* w_out, hipError_t* err) {
  if (w_out || v.K % 2048 || v.N % (SIMT_WAVES * SIMT_R)) return false;
  if ((((uintptr_t)v.q | (uintptr_t)x) & 15) || ((uintptr_t)c & 3)) return false;
  const int steps = v.K / 2048;
  if (steps * MT > 8) return false;  // LDS: MT * K halves, at most 32 KiB
  switch (steps) {
    case 1: *err = launch_unrolled<MX, MT, 1>(v, x, c, M, s); return true;
    case 2: if constexpr (MT <= 4) { *err = launch_unrolled<MX, MT <= 4 ? MT : 1, 2>(v, x, c, M, s); return true; } return false;
    case 4: if constexpr (MT <= 2) { *err = launch_unrolled<MX, MT <= 2 ? MT : 1, 4>(v, x, c, M, s); return true; } return false;
    default: return false;
  }
}

template <int MX, int MT>
static hipError_t launch_mt(const WView& v, const w4_half* x, w4_half* c, int M,
                            hipStream_t s, w4_half* w_out) {
  constexpr int R = SIMT_R;
  hipError_t uerr = hipSuccess;
  if (try_rows4<MX, MT>(v, x, c, M, s, w_out, &uerr)) return uerr;
  if (try_unrolled<MX, MT>(v, x, c, M, s, w_out, &uerr)) return uerr;
  if (try_ksplit<MX, MT>(v, x, c, M, s, w_out, &uerr)) return uerr;
  const bool fast = (v.K % 32 == 0) && (((uintptr_t)v.q & 15) == 0) &&
                    (w_out == nullptr || ((uintptr_t)w_out & 15) == 0);
  const bool x_vec = (v.K % 8 == 0) && (((uintptr_t)x & 15) == 0);
  const bool gs32 = v.mx || (v.gs % 32 == 0);
  const dim3 grid((unsigned)((v.N + SIMT_WAVES * R - 1) / (SIMT_WAVES * R)),
                  (unsigned)((M + MT - 1) / MT));
  constexpr int KC = SIMT_LDS_HALVES / MT;
  const int kc_len = v.K < KC ? v.K : KC;
  const int groups = (kc_len + 7) / 8;
  const int slots = fast ? ((groups + 255) & ~255) : groups;
  const size_t lds = (size_t)slots * MT * 16;
  const dim3 block(SIMT_WAVES * 64);
  if (fast) {
    if (w_out) {
      if (gs32) simt_fast_kernel<MX, MT, R, true, true><<<grid, block, lds, s>>>(v, x, c, M, w_out, x_vec);
      else simt_fast_kernel<MX, MT, R, true, false><<<grid, block, lds, s>>>(v, x, c, M, w_out, x_vec);
    } else {
      if (gs32) simt_fast_kernel<MX, MT, R, false, true><<<grid, block, lds, s>>>(v, x, c, M, w_out, x_vec);
      else simt_fast_kernel<MX, MT, R, false, false><<<grid, block, lds, s>>>(v, x, c, M, w_out, x_vec);
    }
  } else {
    if (w_out) simt_generic_kernel<MX, MT, R, true><<<grid, block, lds, s>>>(v, x, c, M, w_out, x_vec);
    else simt_generic_kernel<MX, MT, R, false><<<grid, block, lds, s>>>(v, x, c, M, w_out, x_vec);
  }
  return hipGetLastError();
}

template <int MX>
static hipError_t launch_fmt(const WView& v, const w4_half* x, w4_half* c, int M,
                             hipStream_t s, w4_half* w_out) {
  if (M == 1) return launch_mt<MX, 1>(v, x, c, M, s, w_out);
  if (M == 2) return launch_mt<MX, 2>(v, x, c, M, s, w_out);
  if (M <= 4) return launch_mt<MX, 4>(v, x, c, M, s, w_out);
  return launch_mt<MX, 8>(v, x, c, M, s, w_out);
}

hipError_t launch_gemm_simt(const WView& v, const w4_half* x, w4_half* c, int M,
                            hipStream_t s, w4_half* w_out) {
  return v.mx ? launch_fmt<1>(v, x, c, M, s, w_out) : launch_fmt<0>(v, x, c, M, s, w_out);
}

}  // namespace w4k
