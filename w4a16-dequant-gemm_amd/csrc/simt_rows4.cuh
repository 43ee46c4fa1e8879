// The decode-shape vector kernel of gemm_simt.hip, in a header of its own so that
// the benchmark's probe library can instantiate its time-stamped form.
#pragma once

#include <utility>

#include "dq.cuh"
#include "../../include/w4_abi.h"

namespace w4k {

constexpr int SIMT_WAVES = 4;  // waves per workgroup of the vector kernels

// ---- decode shapes, four rows per wave -----------------------------------------------
// K = STEPS * 2048, N a multiple of 16, one group per 32-k lane slice with a
// power-of-two group size (or MXFP4), no hook.  What a launch of this size spends
// its time on, measured with time stamps inside the waves (N = K = 4096): 0.25 us
// until the first request leaves a wave (argument fetch, address arithmetic), 0.4 us
// until the first weights arrive, then 17 vector instructions per packed word on one
// wave per SIMD -- as long as the stream itself -- and a reduce-and-store tail.
// Hence:
//  * every argument is a scalar or a pointer, so they arrive in SGPRs with the wave
//    (the build preloads the kernarg segment) instead of through a scalar load;
//  * 256 workgroups of 4 waves x 4 rows: one wave per SIMD, half the waves to
//    launch, and the activations cross L2 -> CU once per 16 rows (through LDS, two
//    16-byte loads per lane and one barrier, both under the latency of the weights);
//  * the scales (and zero-point words) of a wave's four rows are one contiguous run:
//    one load per lane into the wave's own LDS region instead of 4 * STEPS gathers,
//    each with its own address arithmetic, in front of the weight requests;
//  * requests go out in the order activations, scales, weights (memory returns them
//    in that order) and every 1 KiB of a row is expanded as soon as it has landed
//    (hand-placed vmcnt waits), so arithmetic overlaps the rest of the stream.
// The order of additions is that of simt_fast_kernel / simt_unrolled_kernel (one
// chain per lane over steps, words and pairs, then the DPP wave sum): same bytes.
#define W4_GLOAD16_NT(dst, ptr) asm volatile("global_load_dwordx4 %0, %1, off nt" : "=v"(dst) : "v"(ptr) : "memory")
#define W4_GLOAD16(dst, ptr) asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(dst) : "v"(ptr) : "memory")
#define W4_GLOAD4(dst, ptr) asm volatile("global_load_dword %0, %1, off" : "=v"(dst) : "v"(ptr) : "memory")

template <int CNT>
__device__ __forceinline__ void vm_wait() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(CNT) : "memory");
}
// The register was written by an asm load; from here on the compiler may read it.
template <class T>
__device__ __forceinline__ void landed(T& v) {
  asm volatile("" : "+v"(v)::"memory");
}

constexpr int ROWS4_R = 4;

// 100 MHz device clock (10 ns ticks), the same on every compute die.
__device__ __forceinline__ uint64_t rows4_now() {
  uint64_t t;
  asm volatile("s_memrealtime %0\n\ts_waitcnt lgkmcnt(0)" : "=s"(t)::"memory");
  return t;
}
constexpr int ROWS4_STAMPS = 24;  // uint64 slots per wave when TL is set

// TL: every wave records when it started, had issued its requests, saw its
// activations / first weights land, finished each step and the reduction
// (stamps[wave * ROWS4_STAMPS + ...], for the benchmark's timeline probe only).
template <int MX, int MT, int STEPS, bool ASYM, int GSH, bool TL>
__global__ __launch_bounds__(SIMT_WAVES * 64) void simt_rows4_kernel(
    const uint32_t* __restrict__ q, const void* __restrict__ scales,
    const uint32_t* __restrict__ zeros, const w4_half* __restrict__ x, w4_half* __restrict__ c,
    const int N, const int M, const int gs_any, const int G_any, uint64_t* __restrict__ stamps) {
  uint64_t ts[ROWS4_STAMPS];
  if (TL) ts[0] = rows4_now();
  constexpr int R = ROWS4_R, K = STEPS * 2048, WPR = K / 8, NQ = R * STEPS;
  // GSH 5..8: gs = 1 << GSH, one group per 32-k slice.  GSH 0 / 3: any gs % 8 == 0 with
  // gs >= 32 / gs >= 8 (gs_any, G_any groups per row): a group per packed word; the
  // arrays and load counts below are sized for the most groups a row can have.
  constexpr bool ANY = !MX && GSH < 5;
#ifndef W4_ROWS4_FOLD
#define W4_ROWS4_FOLD 1
#endif
  // W4: scale and zero-point applied per group, in FP32 (w4_dot_biased).  Where it pays:
  // with three or four activation rows the dot products dominate a word (16 of 21 - 29
  // instructions) and the per-row bias sums (two per group with zero-points) cost what
  // the shorter expansion saves -- N = K = 4096, M = 4: gs = 128 4.75 -> 4.41 us
  // symmetric but 4.77 -> 4.92 with zero-points, gs = 48 with zero-points 5.63 -> 6.19.
  constexpr bool FOLD = W4_ROWS4_FOLD && !MX &&
                        (ANY ? (ASYM ? MT == 1 : MT <= 2) : (ASYM ? MT <= 2 : true));
  constexpr int PW = ANY ? 4 : 1;                         // bias sums kept per packed word / per 32-k slice
  // Where the bias sums are formed: by the threads that stage the activations (once per
  // workgroup, before the barrier), or by every lane from its own registers at the head
  // of a 2048-k block.  With zero-points (two sums per slice) and one group per slice the
  // second is faster by 2 - 4 % (N = 11008, gs = 128, M = 1 / 2: 5.46 / 6.48 against
  // 5.55 / 6.74 us): it adds nothing in front of the barrier.
  constexpr bool STAGED = FOLD && (ANY || !ASYM);
  constexpr int NG = ANY ? 4 : 1;                         // group lookups per slice
  constexpr int GCAP = MX ? K / 32 : ANY ? (K >> (GSH == 0 ? 5 : 3)) : (K >> GSH);
  const int G = ANY ? G_any : GCAP;                       // groups (blocks) per row
  const int SD = MX ? R * G / 4 : R * G / 2;              // scale dwords of a wave's rows
  constexpr int NSL = ((MX ? R * GCAP / 4 : R * GCAP / 2) + 63) / 64;  // scale loads per lane
  constexpr int WGCAP = (GCAP + 7) / 8;
  const int WG = (G + 7) / 8;                             // zero-point words per row
  constexpr int NZL = ASYM ? (R * WGCAP + 63) / 64 : 0;   // zero-point loads per lane
  constexpr int XL = MT * STEPS;                          // activation loads per thread
  __shared__ u4 xs[MT * STEPS * 256];
  __shared__ uint32_t ss[SIMT_WAVES][NSL * 64];
  __shared__ uint32_t zs[SIMT_WAVES][ASYM ? NZL * 64 : 1];
  __shared__ float xb[STAGED ? MT * STEPS * 64 * PW : 1];          // sum of x_k * bias_k (symmetric: bias_k + 8)
  __shared__ float xa[STAGED && ASYM ? MT * STEPS * 64 * PW : 1];  // sum of x_k
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n0 = (blockIdx.x * SIMT_WAVES + wave) * R;
  const int m0 = blockIdx.y * MT;

  u4 xv[XL], qw[NQ];
  uint32_t sw[NSL], zw[ASYM ? NZL : 1];
#pragma unroll
  for (int t = 0; t < XL; ++t) {
    const int i = t * SIMT_WAVES * 64 + threadIdx.x;
    const int m = min(i / (STEPS * 256), M - 1 - m0), g8 = i % (STEPS * 256);
    W4_GLOAD16(xv[t], x + (size_t)(m0 + m) * K + g8 * 8);  // rows past M: a valid row, never stored
  }
  const uint32_t* srun = (const uint32_t*)((const uint8_t*)scales + (size_t)n0 * (MX ? G : 2 * G));
#pragma unroll
  for (int t = 0; t < NSL; ++t) {
    const int i = min(t * 64 + lane, SD - 1);
    W4_GLOAD4(sw[t], srun + i);
  }
#pragma unroll
  for (int t = 0; t < NZL; ++t) {
    const int i = min(t * 64 + lane, R * WG - 1);
    W4_GLOAD4(zw[t], zeros + (size_t)n0 * WG + i);
  }
#pragma unroll
  for (int i = 0; i < NQ; ++i) {  // block-major: the four rows of a 2048-k block share its activations
    const int st = i / R, r = i % R;
    W4_GLOAD16_NT(qw[i], q + (size_t)(n0 + r) * WPR + st * 256 + lane * 4);
    // The four waves place their runs in step: a barrier after every request.  Memory
    // serves requests roughly in the order they were made; a wave that placed all its
    // requests at once got all its runs late when it came late, with all of its
    // arithmetic still ahead (the slowest wave ended 0.6 us after the median one).
    // Round by round, every wave's run i lands at about the same time and the
    // arithmetic keeps pace with the stream (C1: 3.63 - 3.72 -> 3.50 us in the same runs).
    // With three or four activation rows a wave has enough arithmetic per run to keep
    // up by itself, and the barriers cost (N = 11008: 9.3 -> 9.1 us without them).
    if (MT <= 2 && i + 1 < NQ) asm volatile("s_barrier" ::: "memory");
  }

  if (TL) ts[1] = rows4_now();
  vm_wait<NQ + NZL + NSL>();  // activations
  if (TL) ts[2] = rows4_now();
#pragma unroll
  for (int t = 0; t < XL; ++t) {
    landed(xv[t]);
    const int i = t * SIMT_WAVES * 64 + threadIdx.x;
    const int m = i / (STEPS * 256), g8 = i % (STEPS * 256);
    const int slot = (g8 & ~255) + (g8 & 3) * 64 + ((g8 & 255) >> 2);
    const u4 px = MX ? xv[t] : pair_strided(xv[t]);
    xs[m * STEPS * 256 + slot] = px;
    if constexpr (STAGED) {
      // What the biased codes add to a dot product does not depend on the row: the
      // thread that stages a word's eight activations sums them against the biases
      // here, under the latency of the weights (even k: 1024, odd k: 64; with z = 8
      // for every group the zero-point rides along), and a quad of lanes adds up a slice.
      float vb = 0.0f, va = 0.0f;
      w4_bias_sums<ASYM>(px, vb, va);
      if (ANY) {
        xb[m * STEPS * 256 + slot] = vb;
        if (ASYM) xa[m * STEPS * 256 + slot] = va;
      } else {
        vb = dpp_add<0xB1, 0xF>(vb);
        vb = dpp_add<0x4E, 0xF>(vb);
        if (ASYM) {
          va = dpp_add<0xB1, 0xF>(va);
          va = dpp_add<0x4E, 0xF>(va);
        }
        if ((threadIdx.x & 3) == 0) {  // g8 & 3 == threadIdx.x & 3: the quad is one lane's slice
          xb[m * STEPS * 64 + (g8 >> 8) * 64 + ((g8 & 255) >> 2)] = vb;
          if (ASYM) xa[m * STEPS * 64 + (g8 >> 8) * 64 + ((g8 & 255) >> 2)] = va;
        }
      }
    }
  }
  vm_wait<NQ>();  // scales and zero-points: into this wave's own LDS region
#pragma unroll
  for (int t = 0; t < NSL; ++t) {
    landed(sw[t]);
    ss[wave][t * 64 + lane] = sw[t];
  }
#pragma unroll
  for (int t = 0; t < NZL; ++t) {
    landed(zw[t]);
    zs[wave][t * 64 + lane] = zw[t];
  }
  __syncthreads();

  // group parameters of this lane's slices, read back from LDS
  uint32_t sc[NQ][NG];
  int zp[NQ][NG];
  float sf[FOLD ? NQ : 1][NG], zf[FOLD && ASYM ? NQ : 1][NG];
#pragma unroll
  for (int i = 0; i < NQ; ++i) {
    const int st = i / R, r = i % R;
    int g4[4];
    if (ANY) groups_of_slice(st * 2048 + lane * 32, gs_any, -1, G - 1, g4);
    else g4[0] = MX ? st * 64 + lane : (st * 2048 + lane * 32) >> GSH;
#pragma unroll
    for (int j = 0; j < NG; ++j) {
      const int g = g4[j];
      if (MX) sc[i][j] = ((const uint8_t*)ss[wave])[r * G + g];
      else sc[i][j] = ((const uint16_t*)ss[wave])[r * G + g];
      zp[i][j] = ASYM ? (int)((zs[wave][r * WG + (g >> 3)] >> (4 * (g & 7))) & 0xFu) : 8;
      if constexpr (FOLD) {
        sf[i][j] = half_bits_to_float(sc[i][j]);
        if constexpr (ASYM) zf[i][j] = (float)zp[i][j];
      }
    }
  }

  float acc[R][MT];
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int m = 0; m < MT; ++m) acc[r][m] = 0.0f;
  if (TL) ts[3] = rows4_now();

  // step i expands the 1 KiB run (2048-k block i / R, row i % R); the runs were
  // requested in this order, so run i has landed when at most NQ - 1 - i are outstanding
  u4 xr[MT][4];
  float pb[MT][PW], pa[MT][PW];  // FOLD: this lane's bias sums of the current block
  auto step = [&](auto ic) {
    constexpr int i = decltype(ic)::value;
    constexpr int st = i / R, r = i % R;
    __builtin_amdgcn_sched_barrier(0);
    if (r == 0) {
#pragma unroll
      for (int m = 0; m < MT; ++m)
#pragma unroll
        for (int j = 0; j < 4; ++j) xr[m][j] = xs[m * STEPS * 256 + st * 256 + j * 64 + lane];
    }
    vm_wait<(NQ - 1 - i > 0 ? NQ - 1 - i : 0)>();
    landed(qw[i]);
    if (TL) ts[4 + i] = rows4_now();
    if constexpr (FOLD) {
      // Nothing of this kernel's result is a dequantized weight (a call with the w_out
      // hook never comes here): biased codes, scale and zero-point applied per group in
      // FP32 (w4_dot_biased): 5 + 4 MT instead of 13 + 4 MT vector instructions per word.
      if (r == 0 && STAGED) {
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
          for (int j = 0; j < PW; ++j) {
            const int at = ANY ? m * STEPS * 256 + st * 256 + j * 64 + lane : m * STEPS * 64 + st * 64 + lane;
            pb[m][j] = xb[at];
            if (ASYM) pa[m][j] = xa[at];
          }
      }
      if (r == 0 && !STAGED) {
#pragma unroll
        for (int m = 0; m < MT; ++m) {
          pb[m][0] = pa[m][0] = 0.0f;
#pragma unroll
          for (int j = 0; j < 4; ++j) w4_bias_sums<ASYM>(xr[m][j], pb[m][0], pa[m][0]);
        }
      }
      float t[MT];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int jg = ANY ? j : 0;
        if (ANY || j == 0) {
#pragma unroll
          for (int m = 0; m < MT; ++m)
            t[m] = ASYM ? -__builtin_fmaf(zf[ASYM ? i : 0][jg], pa[m][jg], pb[m][jg]) : -pb[m][jg];
        }
#pragma unroll
        for (int m = 0; m < MT; ++m) t[m] = w4_dot_biased(qw[i][j], xr[m][j], t[m]);
        if (ANY || j == 3) {
#pragma unroll
          for (int m = 0; m < MT; ++m) acc[r][m] = __builtin_fmaf(sf[i][jg], t[m], acc[r][m]);
        }
      }
      return;
    }
    const float mxs = mx_scale(sc[i][0]);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      h2 d[4];
      if (MX) dq_mx(qw[i][j], mxs, d);
      else dq_w4(qw[i][j], w4_group((uint16_t)sc[i][ANY ? j : 0], zp[i][ANY ? j : 0]), d);
#pragma unroll
      for (int m = 0; m < MT; ++m)
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[r][m] = dot2(d[e], as_h2(xr[m][j][e]), acc[r][m]);
    }
  };
  // (a row's chain still runs over its blocks in ascending k, as in the other kernels)
#define W4_STEP(I) \
  if constexpr (I < NQ) step(std::integral_constant<int, I>{});
  W4_STEP(0) W4_STEP(1) W4_STEP(2) W4_STEP(3) W4_STEP(4) W4_STEP(5) W4_STEP(6) W4_STEP(7)
  W4_STEP(8) W4_STEP(9) W4_STEP(10) W4_STEP(11) W4_STEP(12) W4_STEP(13) W4_STEP(14) W4_STEP(15)
#undef W4_STEP
  static_assert(NQ <= 16 && 6 + NQ < ROWS4_STAMPS, "steps are spelled out up to 16");

  if (TL) {
    __builtin_amdgcn_sched_barrier(0);
    ts[4 + NQ] = rows4_now();
  }
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int m = 0; m < MT; ++m) acc[r][m] = wave_sum_to_lane63(acc[r][m]);
  if (TL) {
    __builtin_amdgcn_sched_barrier(0);
    ts[5 + NQ] = rows4_now();
    if (lane == 0) {
      uint64_t* o = stamps + (size_t)(blockIdx.x * SIMT_WAVES + wave) * ROWS4_STAMPS;
#pragma unroll
      for (int i = 0; i < 6 + NQ; ++i) o[i] = ts[i];
      uint32_t xcc;
      asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc));
      o[ROWS4_STAMPS - 1] = xcc & 0xF;
    }
  }
  if (lane == 63) {
#pragma unroll
    for (int m = 0; m < MT; ++m) {
      if (m0 + m >= M) continue;
      uint16_t h[R];
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const _Float16 v = (_Float16)acc[r][m];
        h[r] = __builtin_bit_cast(uint16_t, v);
      }
      // N is a multiple of 16 and c is 8-byte aligned: the four rows leave as one store
      *(u2*)(c + (size_t)(m0 + m) * N + n0) =
          u2{(uint32_t)h[0] | ((uint32_t)h[1] << 16), (uint32_t)h[2] | ((uint32_t)h[3] << 16)};
    }
  }
}
#undef W4_GLOAD16_NT
#undef W4_GLOAD16
#undef W4_GLOAD4

}  // namespace w4k

