// Fused dequant + GEMM on the vector ALUs: c[m,n] = sum_k x[m,k] * W[n,k] with
// W streamed once from HBM as packed 4-bit codes and expanded in VGPRs.
//
// Mapping (wave64): a wave owns R weight rows; per step each lane fetches one
// dwordx4 of each row (4 packed words = 32 consecutive k, 1 KiB per row per
// wave, fully coalesced) and the matching 32 activations of each of the MT
// activation rows from LDS.  Products are v_dot2_f32_f16 into FP32
// accumulators; the K reduction is finished with a cross-lane sum.
//
// Activations are staged in LDS once per workgroup, already pair-permuted to
// line up with the strided pairs dq_*() produces, and laid out so that lane l
// reads 16-byte slot (j*64 + l): consecutive lanes hit consecutive banks.
//
// The FAST path needs 16-byte-aligned rows (K % 32 == 0, aligned bases).
// Otherwise lanes walk single words (ragged K, K = 4104, 72, 100 ...).
#include "dq.cuh"
#include "kernels.h"

namespace w4k {

constexpr int SIMT_WAVES = 4;     // waves per workgroup
constexpr int SIMT_LDS_HALVES = 16384;  // activations resident in LDS at once (32 KiB)

// Stage x[m0 .. m0+MT)[kc .. kc+KC) into LDS, zero-filled past M and K.
// FAST: slot of 8-group g8 (within a 2048-k block) is (g8 & 3) * 64 + (g8 >> 2).
template <int MT, bool FAST>
__device__ __forceinline__ void stage_x(u4* xs, const w4_half* __restrict__ x, int M,
                                        int K, int m0, int kc, int kc_len,
                                        bool x_vec) {
  const int groups = (kc_len + 7) >> 3;  // 8-groups in this chunk
  const int slots = FAST ? ((groups + 255) & ~255) : groups;
  for (int i = threadIdx.x; i < slots * MT; i += SIMT_WAVES * 64) {
    const int m = i / slots, g8 = i - m * slots;
    const int row = m0 + m;
    const int k = kc + g8 * 8;
    u4 v = {0u, 0u, 0u, 0u};
    if (row < M && g8 < groups) {
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
    int slot = g8;
    if (FAST) slot = (g8 & ~255) + (g8 & 3) * 64 + ((g8 & 255) >> 2);
    xs[m * slots + slot] = pair_strided(v);
  }
}

template <int MX, int MT, int R, bool HOOK, bool FAST>
__global__ __launch_bounds__(SIMT_WAVES * 64) void simt_kernel(
    const WView p, const w4_half* __restrict__ x, w4_half* __restrict__ c, const int M,
    w4_half* __restrict__ w_out, const bool x_vec) {
  extern __shared__ u4 xs[];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n0 = (blockIdx.x * SIMT_WAVES + wave) * R;
  const int m0 = blockIdx.y * MT;
  const int wpr = words(p.K);
  const bool hook = HOOK && blockIdx.y == 0;
  const int wg = MX ? 0 : words(p.G);
  const bool gs32 = MX || (p.gs & 31) == 0;  // one group per 32-k lane slice

  float acc[R][MT];
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int m = 0; m < MT; ++m) acc[r][m] = 0.0f;

  constexpr int KC = SIMT_LDS_HALVES / MT;  // k range staged per pass
  for (int kc = 0; kc < p.K; kc += KC) {
    const int kc_len = min(KC, p.K - kc);
    const int groups = (kc_len + 7) >> 3;
    const int slots = FAST ? ((groups + 255) & ~255) : groups;
    if (kc) __syncthreads();
    stage_x<MT, FAST>(xs, x, M, p.K, m0, kc, kc_len, x_vec);
    __syncthreads();
    if (n0 >= p.N) continue;  // wave-uniform; the barriers above stay matched

    if (FAST) {
      // lane slice: words [4*(blk*64 + lane), +4) of the chunk
      for (int blk = 0; blk * 256 < groups; ++blk) {
        const int g8 = blk * 256 + lane * 4;  // first 8-group of this lane
        if (g8 >= groups) break;
        const int k0 = kc + g8 * 8;
        u4 qw[R];
#pragma unroll
        for (int r = 0; r < R; ++r) {
          const int n = min(n0 + r, p.N - 1);
          qw[r] = __builtin_nontemporal_load(
              (const u4*)(p.q + (size_t)n * wpr + (k0 >> 3)));
        }
        u4 xr[MT][4];
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
          for (int j = 0; j < 4; ++j) xr[m][j] = xs[m * slots + blk * 256 + j * 64 + lane];

#pragma unroll
        for (int r = 0; r < R; ++r) {
          const int n = min(n0 + r, p.N - 1);
          W4Group grp;
          MxBlock mb;
          bool any_wide = false;
          if (MX) {
            mb = mx_block(((const uint8_t*)p.scales)[(size_t)n * p.B + (k0 >> 5)]);
            any_wide = __builtin_amdgcn_ballot_w64(mb.wide) != 0;
          } else if (gs32) {
            const int g = k0 / p.gs;
            const int z = p.symmetric ? 8
                                      : (int)((p.zeros[(size_t)n * wg + (g >> 3)] >>
                                               (4 * (g & 7))) & 0xF);
            grp = w4_group(((const uint16_t*)p.scales)[(size_t)n * p.G + g], z);
          }
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            h2 d[4];
            if (MX) {
              dq_mx(qw[r][j], mb, any_wide, d);
            } else {
              if (!gs32) {
                const int g = (k0 + 8 * j) / p.gs;
                const int z = p.symmetric ? 8
                                          : (int)((p.zeros[(size_t)n * wg + (g >> 3)] >>
                                                   (4 * (g & 7))) & 0xF);
                grp = w4_group(((const uint16_t*)p.scales)[(size_t)n * p.G + g], z);
              }
              dq_w4(qw[r][j], grp, d);
            }
#pragma unroll
            for (int m = 0; m < MT; ++m)
#pragma unroll
              for (int i = 0; i < 4; ++i)
                acc[r][m] = dot2(d[i], as_h2(xr[m][j][i]), acc[r][m]);
            if (hook && n0 + r < p.N) {
              h2 nat[4];
              to_natural(d, nat);
              *(u4*)(w_out + (size_t)n * p.K + k0 + 8 * j) =
                  u4{as_u32(nat[0]), as_u32(nat[1]), as_u32(nat[2]), as_u32(nat[3])};
            }
          }
        }
      }
    } else {
      // one word per lane per step; any K, any alignment
      for (int wi = lane; wi < groups; wi += 64) {
        const int k0 = kc + wi * 8;
        u4 xr[MT];
#pragma unroll
        for (int m = 0; m < MT; ++m) xr[m] = xs[m * slots + wi];
#pragma unroll
        for (int r = 0; r < R; ++r) {
          const int n = min(n0 + r, p.N - 1);
          const uint32_t qw = p.q[(size_t)n * wpr + (k0 >> 3)];
          h2 d[4];
          if (MX) {
            const MxBlock mb =
                mx_block(((const uint8_t*)p.scales)[(size_t)n * p.B + (k0 >> 5)]);
            dq_mx(qw, mb, true, d);
          } else {
            const int g = k0 / p.gs;
            const int z = p.symmetric ? 8
                                      : (int)((p.zeros[(size_t)n * wg + (g >> 3)] >>
                                               (4 * (g & 7))) & 0xF);
            dq_w4(qw, w4_group(((const uint16_t*)p.scales)[(size_t)n * p.G + g], z), d);
          }
#pragma unroll
          for (int m = 0; m < MT; ++m)
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[r][m] = dot2(d[i], as_h2(xr[m][i]), acc[r][m]);
          if (hook && n0 + r < p.N) {
            h2 nat[4];
            to_natural(d, nat);
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
  }

  if (n0 >= p.N) return;
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int m = 0; m < MT; ++m) acc[r][m] = wave_sum(acc[r][m]);
  if (lane == 0) {
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

template <int MX, int MT, int R>
static hipError_t launch_mt(const WView& v, const w4_half* x, w4_half* c, int M,
                            hipStream_t s, w4_half* w_out) {
  const bool fast = (v.K % 32 == 0) && (((uintptr_t)v.q & 15) == 0) &&
                    (w_out == nullptr || ((uintptr_t)w_out & 15) == 0);
  const bool x_vec = (v.K % 8 == 0) && (((uintptr_t)x & 15) == 0);
  const dim3 grid((unsigned)((v.N + SIMT_WAVES * R - 1) / (SIMT_WAVES * R)),
                  (unsigned)((M + MT - 1) / MT));
  constexpr int KC = SIMT_LDS_HALVES / MT;
  const int kc_len = v.K < KC ? v.K : KC;
  const int groups = (kc_len + 7) / 8;
  const int slots = fast ? ((groups + 255) & ~255) : groups;
  const size_t lds = (size_t)slots * MT * 16;
#define W4_GO(HOOK, FAST)                                                     \
  simt_kernel<MX, MT, R, HOOK, FAST>                                          \
      <<<grid, SIMT_WAVES * 64, lds, s>>>(v, x, c, M, w_out, x_vec)
  if (w_out) {
    if (fast) W4_GO(true, true); else W4_GO(true, false);
  } else {
    if (fast) W4_GO(false, true); else W4_GO(false, false);
  }
#undef W4_GO
  return hipGetLastError();
}

template <int MX>
static hipError_t launch_fmt(const WView& v, const w4_half* x, w4_half* c, int M,
                             hipStream_t s, w4_half* w_out) {
  if (M == 1) return launch_mt<MX, 1, 2>(v, x, c, M, s, w_out);
  if (M == 2) return launch_mt<MX, 2, 2>(v, x, c, M, s, w_out);
  if (M <= 4) return launch_mt<MX, 4, 2>(v, x, c, M, s, w_out);
  return launch_mt<MX, 8, 2>(v, x, c, M, s, w_out);
}

hipError_t launch_gemm_simt(const WView& v, const w4_half* x, w4_half* c, int M,
                            hipStream_t s, w4_half* w_out) {
  return v.mx ? launch_fmt<1>(v, x, c, M, s, w_out) : launch_fmt<0>(v, x, c, M, s, w_out);
}

}  // namespace w4k
