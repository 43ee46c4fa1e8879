// Fused dequant + GEMM on the matrix cores (v_mfma_f32_16x16x32_f16).
//
// One packed word -- 8 consecutive k of one weight row -- is exactly one lane's
// A operand of a 16x16x32 MFMA (lane l: row l%16, k-block l/16).  A lane loads
// a dwordx4 (4 words of its row), expands each word in VGPRs and feeds four
// MFMAs; packed W never passes through LDS and FP16 W never exists in memory.
// The contraction order inside a 128-k chunk is permuted (MFMA j takes word j
// of every lane, i.e. k-block 4*(l/16)+j); the B operand reads the activations
// with the same permutation, so the sum is unchanged.
//
// D = A*B gives lane l the outputs (n = 4*(l/16)+i, m = l%16): four consecutive
// n of one activation row, stored as one 8-byte write.
//
// Skinny kernel (this file's first kernel): a workgroup owns 16 weight rows and
// up to 64 activation rows; its 4 waves split K chunk-wise and combine through
// LDS in a fixed order, so results are deterministic and every CU streams W
// even when N/16 is only a few hundred.
#include "dq.cuh"
#include "kernels.h"

namespace w4k {

constexpr int MMA_WAVES = 4;
constexpr int MMA_CHUNK = 128;  // k per lane-load step (16 words per row)

__device__ __forceinline__ h8 pack_h8(const h2 n[4]) {
  return h8{n[0][0], n[0][1], n[1][0], n[1][1], n[2][0], n[2][1], n[3][0], n[3][1]};
}

// 8 activations x[m][k .. k+8), zero past M / K.
template <bool XVEC>
__device__ __forceinline__ h8 load_x8(const w4_half* __restrict__ x, int M, int K, int m,
                                      int k) {
  u4 v = {0u, 0u, 0u, 0u};
  if (m < M && k < K) {
    const uint16_t* src = x + (size_t)m * K + k;
    if (XVEC) {
      v = *(const u4*)src;
    } else {
      uint16_t t[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) t[j] = (k + j < K) ? src[j] : (uint16_t)0;
      v = u4{t[0] | ((uint32_t)t[1] << 16), t[2] | ((uint32_t)t[3] << 16),
             t[4] | ((uint32_t)t[5] << 16), t[6] | ((uint32_t)t[7] << 16)};
    }
  }
  return __builtin_bit_cast(h8, v);
}

template <int MX, int MTILES, bool HOOK, bool FAST>
__global__ __launch_bounds__(MMA_WAVES * 64) void mfma_skinny_kernel(
    const WView p, const w4_half* __restrict__ x, w4_half* __restrict__ c, const int M,
    w4_half* __restrict__ w_out) {
  __shared__ f4 red[MMA_WAVES - 1][MTILES][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, b = lane >> 4;
  const int n0 = blockIdx.x * 16;
  const int m0 = blockIdx.y * (16 * MTILES);
  const int wpr = words(p.K);
  const int n = min(n0 + r, p.N - 1);
  const bool row_ok = n0 + r < p.N;
  const bool hook = HOOK && blockIdx.y == 0 && row_ok;
  const int wg = MX ? 0 : words(p.G);
  const int nchunks = (p.K + MMA_CHUNK - 1) / MMA_CHUNK;

  f4 acc[MTILES];
#pragma unroll
  for (int t = 0; t < MTILES; ++t) acc[t] = f4{0.f, 0.f, 0.f, 0.f};

  for (int ch = wave; ch < nchunks; ch += MMA_WAVES) {
    const int w0 = ch * 16 + 4 * b;  // first of this lane's 4 words
    u4 qw = {0u, 0u, 0u, 0u};
    if (FAST) {
      qw = __builtin_nontemporal_load((const u4*)(p.q + (size_t)n * wpr + w0));
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (w0 + j < wpr) qw[j] = p.q[(size_t)n * wpr + w0 + j];
    }
    float mxs = 0.0f;
    if (MX) mxs = mx_scale(((const uint8_t*)p.scales)[(size_t)n * p.B + min(w0 >> 2, p.B - 1)]);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int k0 = (w0 + j) * 8;
      h2 d[4], nat[4];
      if (MX) {
        dq_mx(qw[j], mxs, nat);
      } else {
        const int g = min(k0 / p.gs, p.G - 1);
        const int z = p.symmetric ? 8
                                  : (int)((p.zeros[(size_t)n * wg + (g >> 3)] >>
                                           (4 * (g & 7))) & 0xF);
        dq_w4(qw[j], w4_group(((const uint16_t*)p.scales)[(size_t)n * p.G + g], z), d);
        to_natural(d, nat);
      }
      if (hook && k0 < p.K) {
        uint16_t* out = w_out + (size_t)n * p.K + k0;
        if (FAST) {
          *(u4*)out = u4{as_u32(nat[0]), as_u32(nat[1]), as_u32(nat[2]), as_u32(nat[3])};
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e)
            if (k0 + e < p.K) {
              const uint32_t pair = as_u32(nat[e >> 1]);
              out[e] = (uint16_t)((e & 1) ? pair >> 16 : pair & 0xFFFFu);
            }
        }
      }
      const h8 a = pack_h8(nat);
#pragma unroll
      for (int t = 0; t < MTILES; ++t) {
        const h8 bx = load_x8<FAST>(x, M, p.K, m0 + 16 * t + r, k0);
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, bx, acc[t], 0, 0, 0);
      }
    }
  }

  // Fixed-order combine of the four K slices: wave 0 adds waves 1, 2, 3.
  if (wave > 0) {
#pragma unroll
    for (int t = 0; t < MTILES; ++t) red[wave - 1][t][lane] = acc[t];
  }
  __syncthreads();
  if (wave == 0) {
#pragma unroll
    for (int t = 0; t < MTILES; ++t) {
      f4 s = acc[t];
#pragma unroll
      for (int w = 0; w < MMA_WAVES - 1; ++w) s += red[w][t][lane];
      const int m = m0 + 16 * t + r;  // activation row of this lane
      const int nn = n0 + 4 * b;      // first of its 4 weight rows
      if (m < M) {
        uint16_t hv[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const _Float16 h = (_Float16)s[i];
          hv[i] = __builtin_bit_cast(uint16_t, h);
        }
        uint16_t* dst = c + (size_t)m * p.N + nn;
        if (nn + 3 < p.N && (p.N & 3) == 0 && (((uintptr_t)c & 7) == 0)) {
          *(u2*)dst = u2{hv[0] | ((uint32_t)hv[1] << 16), hv[2] | ((uint32_t)hv[3] << 16)};
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (nn + i < p.N) dst[i] = hv[i];
        }
      }
    }
  }
}

// ---- decode-batch kernel (2 <= M < 96, 16-byte aligned rows) ----------------------
// A workgroup of 8 waves owns 16 * NT weight rows and 16 * MT activation rows;
// wave w owns the w-th eighth of the 128-k chunks of K, walks it CH chunks at a
// time, and the waves combine through LDS in wave order.  A round of a wave issues every load it needs before consuming
// any: scales and zero-points, then the activations (B operands, 64 contiguous
// bytes per lane and chunk, served by L2), then the packed weights (A operands,
// the only HBM stream) -- loads return in issue order, so the weights arrive
// last and nothing waits behind them.  Chunks past K are clamped to k = 0 and
// their activations zeroed, which keeps the round branch-free.
constexpr int DEC_WAVES = 8;

// The four packed words of a lane's 32-k slice starting at word w0 of a row of
// wpr words: one dwordx4 when rows are 16-byte aligned (K % 32 == 0), else four
// dword loads with the index clamped to the row (K % 8 == 0; words past K meet
// zero activations).
template <bool WVEC>
__device__ __forceinline__ u4 load_words4(const uint32_t* __restrict__ row, int w0, int wpr) {
  if (WVEC) return __builtin_nontemporal_load((const u4*)(row + w0));
  u4 v;
#pragma unroll
  for (int j = 0; j < 4; ++j) v[j] = __builtin_nontemporal_load(row + min(w0 + j, wpr - 1));
  return v;
}

template <int FMT, int MT, int NT, int CH, bool HOOK, bool GS32, bool WVEC>
__global__ __launch_bounds__(DEC_WAVES * 64) void mfma_decode_kernel(
    const WView p, const w4_half* __restrict__ x, w4_half* __restrict__ c, const int M,
    w4_half* __restrict__ w_out, const int gs_shift) {
  constexpr bool MX = FMT == 2;
  constexpr int NS = (MX || GS32) ? 1 : 4;  // group lookups per lane and chunk
  __shared__ f4 red[DEC_WAVES][NT * MT][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, b = lane >> 4;
  const int n0 = blockIdx.x * (16 * NT), m0 = blockIdx.y * (16 * MT);
  const int wpr = p.K >> 3;
  const int wg = MX ? 0 : words(p.G);
  const int nchunks = (p.K + MMA_CHUNK - 1) / MMA_CHUNK;
  const bool hook = HOOK && blockIdx.y == 0;

  size_t nrow[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) nrow[t] = (size_t)min(n0 + 16 * t + r, p.N - 1);
  const uint16_t* xrow[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) xrow[mt] = x + (size_t)min(m0 + 16 * mt + r, M - 1) * p.K;

  f4 acc[NT][MT];
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[t][mt] = f4{0.f, 0.f, 0.f, 0.f};

  // wave w owns the chunks [w * cpw, (w + 1) * cpw), walked CH at a time
  const int cpw = (nchunks + DEC_WAVES - 1) / DEC_WAVES;
  const int cend = min(nchunks, (wave + 1) * cpw);
  for (int c0 = wave * cpw; c0 < cend; c0 += CH) {
    int kl[CH];
    bool ok[CH];
    uint32_t sc[CH][NT][NS], zw[CH][NT][NS], zsh[CH][NS];
    u4 xv[CH][MT][4], qw[CH][NT];
#pragma unroll
    for (int i = 0; i < CH; ++i) {
      const int k = (c0 + i) * MMA_CHUNK + b * 32;
      ok[i] = c0 + i < cend && k < p.K;
      kl[i] = ok[i] ? k : 0;
    }
#pragma unroll
    for (int i = 0; i < CH; ++i) {
      int g4[4];
      if (NS == 1) g4[0] = MX ? (kl[i] >> 5) : gs_shift >= 0 ? (kl[i] >> gs_shift) : kl[i] / p.gs;
      else groups_of_slice(kl[i], p.gs, gs_shift, p.G - 1, g4);
#pragma unroll
      for (int e = 0; e < NS; ++e) {
        const int g = g4[e];
        zsh[i][e] = 4u * (uint32_t)(g & 7);
#pragma unroll
        for (int t = 0; t < NT; ++t) {
          if (MX) {
            sc[i][t][e] = ((const uint8_t*)p.scales)[nrow[t] * p.B + g];
          } else {
            sc[i][t][e] = ((const uint16_t*)p.scales)[nrow[t] * p.G + g];
            if (FMT == 1) zw[i][t][e] = p.zeros[nrow[t] * wg + (g >> 3)];
          }
        }
      }
    }
#pragma unroll
    for (int i = 0; i < CH; ++i)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          xv[i][mt][j] = *(const u4*)(xrow[mt] + ((WVEC || kl[i] + 8 * j < p.K) ? kl[i] + 8 * j : 0));
#pragma unroll
    for (int i = 0; i < CH; ++i)
#pragma unroll
      for (int t = 0; t < NT; ++t)
        qw[i][t] = load_words4<WVEC>(p.q + nrow[t] * wpr, kl[i] >> 3, wpr);

#pragma unroll
    for (int i = 0; i < CH; ++i) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          if (!ok[i] || (!WVEC && kl[i] + 8 * j >= p.K)) xv[i][mt][j] = u4{0u, 0u, 0u, 0u};
#pragma unroll
      for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          h2 d[4], nat[4];
          const int e = NS == 1 ? 0 : j;
          if (MX) {
            dq_mx(qw[i][t][j], mx_scale(sc[i][t][0]), nat);
          } else {
            const int z = FMT == 1 ? (int)((zw[i][t][e] >> zsh[i][e]) & 0xFu) : 8;
            dq_w4(qw[i][t][j], w4_group((uint16_t)sc[i][t][e], z), d);
            to_natural(d, nat);
          }
          if (hook && ok[i] && (WVEC || kl[i] + 8 * j < p.K) && n0 + 16 * t + r < p.N)
            *(u4*)(w_out + nrow[t] * p.K + kl[i] + 8 * j) =
                u4{as_u32(nat[0]), as_u32(nat[1]), as_u32(nat[2]), as_u32(nat[3])};
          const h8 a = pack_h8(nat);
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
            acc[t][mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                a, __builtin_bit_cast(h8, xv[i][mt][j]), acc[t][mt], 0, 0, 0);
        }
    }
  }

  // Fixed-order combine of the 8 K slices: wave w sums output tile w.
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) red[wave][t * MT + mt][lane] = acc[t][mt];
  __syncthreads();
  if (wave < NT * MT) {
    f4 s = red[0][wave][lane];
#pragma unroll
    for (int w = 1; w < DEC_WAVES; ++w) s += red[w][wave][lane];
    const int t = wave / MT, mt = wave % MT;
    const int m = m0 + 16 * mt + r;       // activation row of this lane
    const int nn = n0 + 16 * t + 4 * b;   // first of its 4 weight rows
    if (m < M) {
      uint16_t hv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const _Float16 h = (_Float16)s[i];
        hv[i] = __builtin_bit_cast(uint16_t, h);
      }
      uint16_t* dst = c + (size_t)m * p.N + nn;
      if (nn + 3 < p.N && (p.N & 3) == 0 && (((uintptr_t)c & 7) == 0)) {
        *(u2*)dst = u2{hv[0] | ((uint32_t)hv[1] << 16), hv[2] | ((uint32_t)hv[3] << 16)};
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (nn + i < p.N) dst[i] = hv[i];
      }
    }
  }
}

// One chunk per wave and round, one row tile per workgroup: the fastest of the
// (NT, CH) combinations measured for M <= 16 (N = 4096 .. 14336, K = 4096 .. 11008).
template <int FMT, int MT>
static hipError_t launch_decode_mt(const WView& v, const w4_half* x, w4_half* c, int M,
                                   hipStream_t s, w4_half* w_out, bool wvec) {
  const bool gs32 = v.mx || v.gs % 32 == 0;
  int gs_shift = -1;
  if (!v.mx && (v.gs & (v.gs - 1)) == 0) gs_shift = __builtin_ctz((unsigned)v.gs);
  const dim3 grid((unsigned)((v.N + 15) / 16), (unsigned)((M + 16 * MT - 1) / (16 * MT)));
#define W4_GO(HOOK, GS)                                                                       \
  do {                                                                                        \
    if (wvec)                                                                                 \
      mfma_decode_kernel<FMT, MT, 1, 1, HOOK, GS, true>                                       \
          <<<grid, DEC_WAVES * 64, 0, s>>>(v, x, c, M, w_out, gs_shift);                      \
    else                                                                                      \
      mfma_decode_kernel<FMT, MT, 1, 1, HOOK, GS, false>                                      \
          <<<grid, DEC_WAVES * 64, 0, s>>>(v, x, c, M, w_out, gs_shift);                      \
  } while (0)
  if (w_out) {
    if (gs32) W4_GO(true, true); else W4_GO(true, false);
  } else {
    if (gs32) W4_GO(false, true); else W4_GO(false, false);
  }
#undef W4_GO
  return hipGetLastError();
}

// Hooked calls of the shapes the resident-activation kernels take with 17 <= M <= 64:
// same K split, same order of additions.  Group lookups (one per slice or one per
// word) and row loads (16-byte or word by word) follow the arguments.
template <int FMT, int MT>
static hipError_t launch_decode_hooked_mt(const WView& v, const w4_half* x, w4_half* c, int M,
                                          hipStream_t s, w4_half* w_out, bool wvec) {
  const bool gs32 = v.mx || v.gs % 32 == 0;
  if (!w_out || v.K % 8 || (((uintptr_t)w_out | (uintptr_t)x) & 15)) return hipErrorInvalidValue;
  int gs_shift = -1;
  if (!v.mx && (v.gs & (v.gs - 1)) == 0) gs_shift = __builtin_ctz((unsigned)v.gs);
  const dim3 grid((unsigned)((v.N + 15) / 16), (unsigned)((M + 16 * MT - 1) / (16 * MT)));
#define W4_GO(GS, WV) \
  mfma_decode_kernel<FMT, MT, 1, 1, true, GS, WV><<<grid, DEC_WAVES * 64, 0, s>>>(v, x, c, M, w_out, gs_shift)
  if (gs32) {
    if (wvec) W4_GO(true, true); else W4_GO(true, false);
  } else {
    if (wvec) W4_GO(false, true); else W4_GO(false, false);
  }
#undef W4_GO
  return hipGetLastError();
}

template <int FMT>
static hipError_t launch_decode(const WView& v, const w4_half* x, w4_half* c, int M,
                                hipStream_t s, w4_half* w_out, bool wvec) {
  if (M <= 16) return launch_decode_mt<FMT, 1>(v, x, c, M, s, w_out, wvec);
  if (M <= 32) return launch_decode_hooked_mt<FMT, 2>(v, x, c, M, s, w_out, wvec);
  return launch_decode_hooked_mt<FMT, 4>(v, x, c, M, s, w_out, wvec);  // grid.y walks 64 rows at a time
}

// ---- streaming decode-batch kernel --------------------------------------------------
// 8 waves = NW row tiles x KW slices of K.  The waves of one K slice share the
// activations of that slice through LDS (staged 128 k at a time, double
// buffered, one barrier per step), so x crosses L2 -> CU once per workgroup
// instead of once per wave; each wave streams its own 16 weight rows straight
// into registers as MFMA A operands, DEPTH steps ahead.  Steps past the end of a
// slice, and k past K, fetch from clamped addresses and stage zeros.
// LEAN: K is a whole number of steps per slice and of ring rounds, N a whole
// number of workgroups, the group size a power of two: every bounds test and
// its branch disappears from the loop (the kernel is bound by instruction issue).
template <int FMT, int MT, int NW, int KW, int CPS, int DEPTH, bool HOOK, bool GS32, bool WVEC,
          bool LEAN>
__global__ __launch_bounds__(64 * NW * KW) void mfma_stream_kernel(
    const WView p, const w4_half* __restrict__ x, w4_half* __restrict__ c, const int M,
    w4_half* __restrict__ w_out, const int gs_shift) {
  constexpr int THREADS = 64 * NW * KW;
  static_assert(!LEAN || (GS32 && WVEC), "lean form: one group per lane slice, aligned rows");
  constexpr bool MX = FMT == 2;
  constexpr int NS = (MX || GS32) ? 1 : 4;
  constexpr int ROWS = 16 * MT;
  constexpr int BK = MMA_CHUNK * CPS;         // k per step
  constexpr int SEGS = BK / 8;                // 16-byte pieces per staged row
  constexpr int LD = BK + 8;                  // halves per staged row: 16-lane reads hit 16 bank groups
  constexpr int PIECES = KW * ROWS * SEGS;    // pieces staged per step
  constexpr int XP = (PIECES + THREADS - 1) / THREADS;  // ... per thread
  constexpr int XS_HALVES = 2 * KW * ROWS * LD;
  constexpr int RED_HALVES = KW * NW * MT * 64 * 8;
  __shared__ __attribute__((aligned(16))) uint16_t smem[XS_HALVES > RED_HALVES ? XS_HALVES : RED_HALVES];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 15, b = lane >> 4;
  const int nw = wave % NW, kw = wave / NW;
  const int n0 = blockIdx.x * (16 * NW) + 16 * nw, m0 = blockIdx.y * ROWS;
  const int wpr = p.K >> 3;
  const int wg = MX ? 0 : words(p.G);
  const int nblocks = (p.K + BK - 1) / BK;
  const int cpk = (nblocks + KW - 1) / KW;                  // steps per K slice
  const int steps = LEAN ? cpk : (cpk + DEPTH - 1) / DEPTH * DEPTH;
  const bool hook = HOOK && blockIdx.y == 0 && n0 + r < p.N;
  const size_t nrow = LEAN ? (size_t)(n0 + r) : (size_t)min(n0 + r, p.N - 1);
  const uint32_t* qrow = p.q + nrow * wpr;

  // the pieces of x this thread stages every step
  const uint16_t* xsrc[XP];  // start of the activation row
  int xk0[XP], xdst[XP];     // first k of the piece at step 0; where it goes in a staging buffer
#pragma unroll
  for (int i = 0; i < XP; ++i) {
    const int id = i * THREADS + tid;
    const int pk = (id / (ROWS * SEGS)) % KW, prow = (id / SEGS) % ROWS, seg = (id % SEGS) * 8;
    xsrc[i] = x + (size_t)min(m0 + prow, M - 1) * p.K;
    xk0[i] = pk * cpk * BK + seg;
    xdst[i] = pk * (ROWS * LD) + prow * LD + seg;
  }

  struct Slot {
    u4 q[CPS];
    uint32_t sc[CPS][NS], zw[CPS][NS], zsh[CPS][NS];
    u4 xg[XP];
  };
  Slot ring[DEPTH];
  auto group_of = [&](int kk) {
    return MX ? (kk >> 5) : (LEAN || gs_shift >= 0) ? (kk >> gs_shift) : kk / p.gs;
  };
  auto lane_k = [&](int s, int ch) { return (kw * cpk + s) * BK + ch * MMA_CHUNK + b * 32; };
  auto fetch = [&](Slot& sl, int s) {
    if (LEAN) s = min(s, cpk - 1);  // the ring runs past the end of the slice: refetch the last step
#pragma unroll
    for (int ch = 0; ch < CPS; ++ch) {
      const int k = lane_k(s, ch);
      const int kc = (LEAN || (s < cpk && k < p.K)) ? k : 0;
      int g[4];
      if (NS == 1) g[0] = group_of(kc);
      else groups_of_slice(kc, p.gs, gs_shift, p.G - 1, g);
#pragma unroll
      for (int e = 0; e < NS; ++e) {
        if (MX) {
          sl.sc[ch][e] = ((const uint8_t*)p.scales)[nrow * p.B + g[e]];
        } else {
          sl.sc[ch][e] = ((const uint16_t*)p.scales)[nrow * p.G + g[e]];
          if (FMT == 1) {
            sl.zw[ch][e] = p.zeros[nrow * wg + (g[e] >> 3)];
            sl.zsh[ch][e] = 4u * (uint32_t)(g[e] & 7);
          }
        }
      }
    }
#pragma unroll
    for (int i = 0; i < XP; ++i) {
      const int kx = xk0[i] + s * BK;
      sl.xg[i] = *(const u4*)(xsrc[i] + ((LEAN || (s < cpk && kx < p.K)) ? kx : 0));
    }
#pragma unroll
    for (int ch = 0; ch < CPS; ++ch) {
      const int k = lane_k(s, ch);
      const int kc = (LEAN || (s < cpk && k < p.K)) ? k : 0;
      sl.q[ch] = load_words4<WVEC>(qrow, kc >> 3, wpr);
    }
  };
  auto stage = [&](const Slot& sl, int buf, int s) {
    uint16_t* base = smem + buf * (KW * ROWS * LD);
#pragma unroll
    for (int i = 0; i < XP; ++i) {
      const int kx = xk0[i] + s * BK;
      const bool okx = LEAN || (s < cpk && kx < p.K);
      // W4: staged in the (k, k+4) pairing the expansion step produces, so the
      // weights need no re-pairing on their way into the MFMA
      if (XP * THREADS == PIECES || i * THREADS + tid < PIECES)
        *(u4*)(base + xdst[i]) = okx ? (MX ? sl.xg[i] : pair_strided(sl.xg[i])) : u4{0u, 0u, 0u, 0u};
    }
  };

  f4 acc[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) acc[mt] = f4{0.f, 0.f, 0.f, 0.f};

#pragma unroll
  for (int d = 0; d < DEPTH; ++d) fetch(ring[d], d);
  stage(ring[0], 0, 0);
  __syncthreads();
  for (int s0 = 0; s0 < steps; s0 += DEPTH) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      const int s = s0 + d, buf = s & 1;
      u4 q[CPS];
      uint32_t sc[CPS][NS], zw[CPS][NS], zsh[CPS][NS];
#pragma unroll
      for (int ch = 0; ch < CPS; ++ch) {
        q[ch] = ring[d].q[ch];
#pragma unroll
        for (int e = 0; e < NS; ++e)
          sc[ch][e] = ring[d].sc[ch][e], zw[ch][e] = ring[d].zw[ch][e], zsh[ch][e] = ring[d].zsh[ch][e];
      }
      fetch(ring[d], s + DEPTH);  // slot d: weights copied out, activations staged one step ago
      stage(ring[(d + 1) % DEPTH], buf ^ 1, s + 1);
      const uint16_t* xb = smem + buf * (KW * ROWS * LD) + kw * (ROWS * LD) + r * LD + b * 32;
#pragma unroll
      for (int ch = 0; ch < CPS; ++ch) {
        const int k = lane_k(s, ch);
        const bool okw = LEAN || (s < cpk && k < p.K);
        const int kc = okw ? k : 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          h2 dq[4];  // MX: natural pairs; W4: (k, k+4) pairs, like the staged activations
          const int e = NS == 1 ? 0 : j;
          if (MX) {
            dq_mx(q[ch][j], mx_scale(sc[ch][0]), dq);
          } else {
            int z = 8;
            if (FMT == 1) z = (int)((zw[ch][e] >> zsh[ch][e]) & 0xFu);
            dq_w4(q[ch][j], w4_group((uint16_t)sc[ch][e], z), dq);
          }
          if (hook && okw && (WVEC || kc + 8 * j < p.K)) {
            h2 nat[4];
            if (MX) {
#pragma unroll
              for (int t = 0; t < 4; ++t) nat[t] = dq[t];
            } else {
              to_natural(dq, nat);
            }
            *(u4*)(w_out + nrow * p.K + kc + 8 * j) =
                u4{as_u32(nat[0]), as_u32(nat[1]), as_u32(nat[2]), as_u32(nat[3])};
          }
          const h8 a = pack_h8(dq);
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) {
            const h8 bx = *(const h8*)(xb + mt * 16 * LD + ch * MMA_CHUNK + j * 8);
            acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, bx, acc[mt], 0, 0, 0);
          }
        }
      }
      __syncthreads();
    }
  }

  // Fixed-order combine of the KW slices (the staging buffers are free now).
  f4* red = (f4*)smem;  // [KW][NW * MT][64]
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) red[(kw * (NW * MT) + nw * MT + mt) * 64 + lane] = acc[mt];
  __syncthreads();
  for (int tile = wave; tile < NW * MT; tile += NW * KW) {
    f4 sum = red[tile * 64 + lane];
#pragma unroll
    for (int w = 1; w < KW; ++w) sum += red[(w * (NW * MT) + tile) * 64 + lane];
    const int m = m0 + 16 * (tile % MT) + r;                              // activation row of this lane
    const int nn = blockIdx.x * (16 * NW) + 16 * (tile / MT) + 4 * b;    // first of its 4 weight rows
    if (m < M) {
      uint16_t hv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const _Float16 h = (_Float16)sum[i];
        hv[i] = __builtin_bit_cast(uint16_t, h);
      }
      uint16_t* dst = c + (size_t)m * p.N + nn;
      if (nn + 3 < p.N && (p.N & 3) == 0 && (((uintptr_t)c & 7) == 0)) {
        *(u2*)dst = u2{hv[0] | ((uint32_t)hv[1] << 16), hv[2] | ((uint32_t)hv[3] << 16)};
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (nn + i < p.N) dst[i] = hv[i];
      }
    }
  }
}


template <int FMT, int MT, int NW, int KW>
static hipError_t launch_stream_cfg(const WView& v, const w4_half* x, w4_half* c, int M,
                                   hipStream_t s, w4_half* w_out, bool wvec) {
  const bool gs32 = v.mx || v.gs % 32 == 0;
  int gs_shift = -1;
  if (!v.mx && (v.gs & (v.gs - 1)) == 0) gs_shift = __builtin_ctz((unsigned)v.gs);
  // two chunks per step, two steps in flight (deeper rings measured slower: 15.2 -> 16-17 us
  // at N = 11008, M = 16); MT = 4 fills the LDS with one chunk per step
  constexpr int CPS = MT == 4 ? 1 : 2;
  constexpr int DEPTH = MT == 4 ? 4 : 2;
  const dim3 grid((unsigned)((v.N + 16 * NW - 1) / (16 * NW)), (unsigned)((M + 16 * MT - 1) / (16 * MT)));
  const int cpk = ((v.K + MMA_CHUNK * CPS - 1) / (MMA_CHUNK * CPS) + KW - 1) / KW;
#define W4_GO(D, HOOK, GS)                                                                    \
  do {                                                                                        \
    if (wvec)                                                                                 \
      mfma_stream_kernel<FMT, MT, NW, KW, CPS, D, HOOK, GS, true, false>                      \
          <<<grid, 64 * NW * KW, 0, s>>>(v, x, c, M, w_out, gs_shift);                                 \
    else                                                                                      \
      mfma_stream_kernel<FMT, MT, NW, KW, CPS, D, HOOK, GS, false, false>                     \
          <<<grid, 64 * NW * KW, 0, s>>>(v, x, c, M, w_out, gs_shift);                                 \
  } while (0)
  // the lean form: whole steps, whole ring rounds, whole workgroups, shift for the group index.
  // Measured at N = 11008, K = 4096: 23.7 vs 25.6 us with four activation tiles (M = 64), but
  // 18.4 vs 15.2 us with one (M = 16) and 19.8 vs 18.4 us with two, so only MT = 4 takes it.
  const bool lean = MT == 4 && wvec && gs32 && (v.mx || gs_shift >= 0) && v.K % (MMA_CHUNK * CPS * KW) == 0 &&
                    v.N % (16 * NW) == 0;
  bool lean_done = false;
  if constexpr (MT == 4) {  // (the lean form is compiled for four activation tiles only)
    if (lean && w_out) {
      mfma_stream_kernel<FMT, MT, NW, KW, CPS, 1, true, true, true, true>
          <<<grid, 64 * NW * KW, 0, s>>>(v, x, c, M, w_out, gs_shift);
      lean_done = true;
    } else if (lean && cpk % DEPTH == 0) {
      mfma_stream_kernel<FMT, MT, NW, KW, CPS, DEPTH, false, true, true, true>
          <<<grid, 64 * NW * KW, 0, s>>>(v, x, c, M, w_out, gs_shift);
      lean_done = true;
    }
  }
  if (lean_done) {
  } else if (w_out) {
    if (gs32) W4_GO(1, true, true); else W4_GO(1, true, false);
  } else if (cpk >= DEPTH) {
    if (gs32) W4_GO(DEPTH, false, true); else W4_GO(DEPTH, false, false);
  } else {
    if (gs32) W4_GO(1, false, true); else W4_GO(1, false, false);
  }
#undef W4_GO
  return hipGetLastError();
}

// 4 row tiles x 2 K slices per workgroup; 2 x 4 when that grid would leave half of the
// chip idle (N = 4096, M = 32: 13.1 vs 16.2 us; K = 11008: 29 vs 38 us).  16 waves
// measured slower.
template <int FMT, int MT>
static hipError_t launch_stream_mt(const WView& v, const w4_half* x, w4_half* c, int M,
                                   hipStream_t s, w4_half* w_out, bool wvec) {
  const long long wgs = (long long)((v.N + 63) / 64) * ((M + 16 * MT - 1) / (16 * MT));
  if constexpr (MT < 4) {
    if (wgs < 128) return launch_stream_cfg<FMT, MT, 2, 4>(v, x, c, M, s, w_out, wvec);
  }
  return launch_stream_cfg<FMT, MT, 4, 2>(v, x, c, M, s, w_out, wvec);
}

template <int FMT>
static hipError_t launch_stream(const WView& v, const w4_half* x, w4_half* c, int M,
                                hipStream_t s, w4_half* w_out, bool wvec) {
  if (M <= 16) return launch_stream_mt<FMT, 1>(v, x, c, M, s, w_out, wvec);
  if (M <= 32) return launch_stream_mt<FMT, 2>(v, x, c, M, s, w_out, wvec);
  return launch_stream_mt<FMT, 4>(v, x, c, M, s, w_out, wvec);
}

// ---- large-M kernel -----------------------------------------------------------
// Workgroup tile 256 (m) x 128 (n), k-step 64, WM x WN waves each owning a
// (256/WM) x (128/WN) sub-tile of 16x16 MFMA tiles.  Both
// operands go through LDS as FP16 in unpadded 128-byte rows whose 16-byte chunks
// are XOR-swizzled by the row pair, so that 16 consecutive lanes -- of the
// operand reads (16 rows, one chunk) and of the staging writes (2 or 4 rows) --
// touch 16 distinct bank groups (the bank-conflict counter fell 4x against rows
// padded to 144 bytes).  The
// packed weights of a k-step are one dwordx2 per thread; they are expanded in
// VGPRs once per workgroup tile (so the dequant cost is amortised over 256
// activation rows) and written to LDS in natural k order.
//
// A k-step of MFMAs is far shorter than an HBM round trip, so DEPTH k-steps are
// kept in flight in registers; LDS is double buffered, one barrier per k-step.
// The loop body is branch-free (rows past M and k-steps past K are clamped to
// valid addresses and their results never stored), which lets the compiler
// retire exactly the loads a k-step needs instead of draining the queue.
//
// Tiles are handed to workgroups so that the workgroups resident on one XCD
// (ids congruent mod 8) walk the n-tiles of the same m-tile: the activation
// slab stays in that XCD's L2 and every weight tile is fetched once per XCD.
constexpr int TB_M = 256, TB_N = 128, TB_K = 64, TB_LD = TB_K;
// 16-byte chunk `chunk` of LDS row `row` lives at chunk ^ ((row >> 1) & 7)
#define W4_SWZ(row, chunk) ((chunk) ^ (((row) >> 1) & 7))

// FMT: 0 W4 symmetric, 1 W4 asymmetric, 2 MXFP4.  WM x WN waves, each a
// (256/WM) x (128/WN) sub-tile.
template <int FMT, bool HOOK, bool GS16, int DEPTH, int WM, int WN>
__global__ __launch_bounds__(WM * WN * 64) void mfma_tile_kernel(
    const WView p, const w4_half* __restrict__ x, w4_half* __restrict__ c, const int M,
    w4_half* __restrict__ w_out, const int tiles_m, const int tiles_n) {
  constexpr bool MX = FMT == 2;
  constexpr int THREADS = WM * WN * 64;
  constexpr int TI = TB_M / WM / 16, TJ = TB_N / WN / 16;  // MFMA tiles per wave
  constexpr int XCH = TB_M * 8 / THREADS;                   // 16-byte activation chunks per thread
  constexpr int WPT = TB_N * 8 / THREADS;                   // packed words per thread (2 or 4)
  constexpr int TPR = 8 / WPT;                              // threads per weight row
  __shared__ __attribute__((aligned(16))) uint16_t xs[2][TB_M * TB_LD];
  __shared__ __attribute__((aligned(16))) uint16_t ws[2][TB_N * TB_LD];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int total = tiles_m * tiles_n, per_xcd = (total + 7) / 8;
  const int t = (int)(blockIdx.x & 7) * per_xcd + (int)(blockIdx.x >> 3);
  if (t >= total) return;
  const int m0 = (t / tiles_n) * TB_M, n0 = (t % tiles_n) * TB_N;
  const int wm = (wave % WM) * (TB_M / WM), wn = (wave / WM) * (TB_N / WN);
  const int wpr = words(p.K);
  const int wg = MX ? 0 : words(p.G);
  const bool hook = HOOK && m0 == 0;
  constexpr int NS = (MX || GS16) ? 1 : WPT;  // GS16: one group per thread's words
  const int nk = p.K / TB_K;

  f4 acc[TI][TJ];
#pragma unroll
  for (int i = 0; i < TI; ++i)
#pragma unroll
    for (int j = 0; j < TJ; ++j) acc[i][j] = f4{0.f, 0.f, 0.f, 0.f};

  // What this thread fetches per k-step: XCH x 16 bytes of activations (row
  // clamped to M-1) and WPT packed words of one weight row (clamped to N-1).
  const int wrow = tid / TPR, wpart = tid % TPR;
  const uint32_t* qrow = p.q + (size_t)min(n0 + wrow, p.N - 1) * wpr + wpart * WPT;
  const size_t srow = (size_t)min(n0 + wrow, p.N - 1);
  const uint16_t* xrow[XCH];
#pragma unroll
  for (int i = 0; i < XCH; ++i) {
    const int id = i * THREADS + tid;
    xrow[i] = x + (size_t)min(m0 + (id >> 3), M - 1) * p.K + (id & 7) * 8;
  }
  struct Slot {
    u4 xg[XCH];
    uint32_t wq[WPT];
    uint32_t wsb[NS], wzw[NS];
  };
  Slot ring[DEPTH];
  auto fetch = [&](Slot& sl, int kt) {
    const int k0 = min(kt, nk - 1) * TB_K;
#pragma unroll
    for (int i = 0; i < XCH; ++i) sl.xg[i] = *(const u4*)(xrow[i] + k0);
    if constexpr (WPT == 4) {
      const u4 v = __builtin_nontemporal_load((const u4*)(qrow + (k0 >> 3)));
#pragma unroll
      for (int j = 0; j < 4; ++j) sl.wq[j] = v[j];
    } else {
      const u2 v = __builtin_nontemporal_load((const u2*)(qrow + (k0 >> 3)));
      sl.wq[0] = v[0];
      sl.wq[1] = v[1];
    }
#pragma unroll
    for (int i = 0; i < NS; ++i) {
      const int w0 = (k0 >> 3) + wpart * WPT + i;
      if (MX) {
        sl.wsb[i] = ((const uint8_t*)p.scales)[srow * p.B + (w0 >> 2)];
      } else {
        const int g = (8 * w0) / p.gs;
        sl.wsb[i] = ((const uint16_t*)p.scales)[srow * p.G + g];
        if (FMT == 1) sl.wzw[i] = p.zeros[srow * wg + (g >> 3)];
      }
    }
  };
  auto stage = [&](const Slot& sl, int buf, int kt) {  // registers -> LDS, weights expanded
    const int k0 = kt * TB_K;
#pragma unroll
    for (int i = 0; i < XCH; ++i) {
      const int id = i * THREADS + tid, row = id >> 3, kc = id & 7;
      *(u4*)(xs[buf] + row * TB_LD + W4_SWZ(row, kc) * 8) = sl.xg[i];
    }
#pragma unroll
    for (int j = 0; j < WPT; ++j) {
      h2 d[4], nat[4];
      if (MX) {
        dq_mx(sl.wq[j], mx_scale(sl.wsb[0]), nat);
      } else {
        const int i = NS == 1 ? 0 : j;
        int z = 8;
        if (FMT == 1) {
          const int g = (k0 + (wpart * WPT + j) * 8) / p.gs;
          z = (int)((sl.wzw[i] >> (4 * (g & 7))) & 0xFu);
        }
        dq_w4(sl.wq[j], w4_group((uint16_t)sl.wsb[i], z), d);
        to_natural(d, nat);
      }
      const u4 v = u4{as_u32(nat[0]), as_u32(nat[1]), as_u32(nat[2]), as_u32(nat[3])};
      *(u4*)(ws[buf] + wrow * TB_LD + W4_SWZ(wrow, wpart * WPT + j) * 8) = v;
      if (hook && n0 + wrow < p.N)
        *(u4*)(w_out + (size_t)(n0 + wrow) * p.K + k0 + (wpart * WPT + j) * 8) = v;
    }
  };

#pragma unroll
  for (int d = 0; d < DEPTH; ++d) fetch(ring[d], d);
  stage(ring[0], 0, 0);
  __syncthreads();
  for (int kt0 = 0; kt0 < nk; kt0 += DEPTH) {  // nk is a multiple of DEPTH
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      const int kt = kt0 + d;
      const int buf = kt & 1;
      fetch(ring[d], kt + DEPTH);  // slot d held k-step kt, which is already in LDS
      __builtin_amdgcn_iglp_opt(0);  // let the scheduler weave LDS traffic between the MFMAs
      // k-step kt+1 goes to the other buffer (a surplus copy of the last k-step
      // on the final iteration: nobody reads it)
      stage(ring[(d + 1) % DEPTH], buf ^ 1, min(kt + 1, nk - 1));
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) {
        h8 a[TJ], b[TI];
        // wm, wn and the 16-row tile offsets are multiples of 16: the swizzle term depends on the lane only
        const int koff = W4_SWZ(lane & 15, kk * 4 + (lane >> 4)) * 8;
#pragma unroll
        for (int j = 0; j < TJ; ++j)
          a[j] = *(const h8*)(ws[buf] + (wn + j * 16 + (lane & 15)) * TB_LD + koff);
#pragma unroll
        for (int i = 0; i < TI; ++i)
          b[i] = *(const h8*)(xs[buf] + (wm + i * 16 + (lane & 15)) * TB_LD + koff);
#pragma unroll
        for (int i = 0; i < TI; ++i)
#pragma unroll
          for (int j = 0; j < TJ; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[j], b[i], acc[i][j], 0, 0, 0);
      }
      __syncthreads();
    }
  }

  // lane holds c[m][n .. n+4) for m = tile row (lane & 15), n = 4 * (lane >> 4)
  const bool vec_ok = (p.N & 3) == 0 && (((uintptr_t)c & 7) == 0);
#pragma unroll
  for (int i = 0; i < TI; ++i) {
    const int m = m0 + wm + i * 16 + (lane & 15);
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < TJ; ++j) {
      const int n = n0 + wn + j * 16 + 4 * (lane >> 4);
      uint16_t hv[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const _Float16 h = (_Float16)acc[i][j][e];
        hv[e] = __builtin_bit_cast(uint16_t, h);
      }
      uint16_t* dst = c + (size_t)m * p.N + n;
      if (vec_ok && n + 3 < p.N) {
        *(u2*)dst = u2{hv[0] | ((uint32_t)hv[1] << 16), hv[2] | ((uint32_t)hv[3] << 16)};
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (n + e < p.N) dst[e] = hv[e];
      }
    }
  }
}

// 4 x 2 waves (64 x 64 outputs each), 4 k-steps in flight: the fastest of the
// (WM, WN, DEPTH) combinations measured at M = 2048 and 4096, N = K = 4096.
#define W4_TILE_WM 4
#define W4_TILE_WN 2
#define W4_TILE_DEPTH 4

template <int FMT, bool HOOK, bool GSOK, int DEPTH>
static hipError_t launch_tile(const WView& v, const w4_half* x, w4_half* c, int M, hipStream_t s,
                              w4_half* w_out, int tiles_m, int tiles_n, unsigned grid) {
  mfma_tile_kernel<FMT, HOOK, GSOK, DEPTH, W4_TILE_WM, W4_TILE_WN>
      <<<grid, W4_TILE_WM * W4_TILE_WN * 64, 0, s>>>(v, x, c, M, w_out, tiles_m, tiles_n);
  return hipGetLastError();
}

template <int FMT>
static hipError_t launch_tile_fmt(const WView& v, const w4_half* x, w4_half* c, int M,
                                  hipStream_t s, w4_half* w_out, int tm, int tn, unsigned grid) {
  constexpr int WPT = TB_N * 8 / (W4_TILE_WM * W4_TILE_WN * 64);
  const bool gsok = v.mx || v.gs % (8 * WPT) == 0;  // one group per thread's words
  const int nk = v.K / TB_K;
  if (w_out)
    return gsok ? launch_tile<FMT, true, true, 1>(v, x, c, M, s, w_out, tm, tn, grid)
                : launch_tile<FMT, true, false, 1>(v, x, c, M, s, w_out, tm, tn, grid);
  if (!gsok) return launch_tile<FMT, false, false, 1>(v, x, c, M, s, w_out, tm, tn, grid);
  if (nk % W4_TILE_DEPTH == 0)
    return launch_tile<FMT, false, true, W4_TILE_DEPTH>(v, x, c, M, s, w_out, tm, tn, grid);
  if (nk % 2 == 0) return launch_tile<FMT, false, true, 2>(v, x, c, M, s, w_out, tm, tn, grid);
  return launch_tile<FMT, false, true, 1>(v, x, c, M, s, w_out, tm, tn, grid);
}

template <int MX>
static bool try_tile(const WView& v, const w4_half* x, w4_half* c, int M, hipStream_t s,
                     w4_half* w_out, hipError_t* err) {
  if (M < 96 || v.K % TB_K) return false;
  if ((((uintptr_t)v.q | (uintptr_t)x) & 15) || (w_out && ((uintptr_t)w_out & 15))) return false;
  const int tiles_m = (M + TB_M - 1) / TB_M, tiles_n = (v.N + TB_N - 1) / TB_N;
  const long long total = (long long)tiles_m * tiles_n;
  if (total > (1LL << 28)) return false;
  const unsigned grid = (unsigned)(8 * ((total + 7) / 8));
  if (MX) *err = launch_tile_fmt<2>(v, x, c, M, s, w_out, tiles_m, tiles_n, grid);
  else if (v.symmetric) *err = launch_tile_fmt<0>(v, x, c, M, s, w_out, tiles_m, tiles_n, grid);
  else *err = launch_tile_fmt<1>(v, x, c, M, s, w_out, tiles_m, tiles_n, grid);
  return true;
}

template <int MX, int MTILES>
static hipError_t launch_tiles(const WView& v, const w4_half* x, w4_half* c, int M,
                               hipStream_t s, w4_half* w_out) {
  const bool fast = (v.K % 32 == 0) && (((uintptr_t)v.q & 15) == 0) &&
                    (((uintptr_t)x & 15) == 0) &&
                    (w_out == nullptr || ((uintptr_t)w_out & 15) == 0);
  const dim3 grid((unsigned)((v.N + 15) / 16),
                  (unsigned)((M + 16 * MTILES - 1) / (16 * MTILES)));
#define W4_GO(HOOK, FAST) \
  mfma_skinny_kernel<MX, MTILES, HOOK, FAST><<<grid, MMA_WAVES * 64, 0, s>>>(v, x, c, M, w_out)
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
  hipError_t terr = hipSuccess;
  // Shapes of the kernel that fetches the activations once per workgroup (M <= 256):
  // hooked calls take the K-split kernel, which adds in the same order.
  const bool wvec = (v.K % 32 == 0) && (((uintptr_t)v.q) & 15) == 0;
  const bool resident = wvec && decode_resident_applies(v, x, c, M) &&
                        (w_out == nullptr || ((uintptr_t)w_out & 15) == 0);
  // long K, M <= 64: the same sums with the requests pipelined chunk by chunk
  const bool longk = wvec && decode_longk_applies(v, x, c, M) &&
                     (w_out == nullptr || ((uintptr_t)w_out & 15) == 0);
  if (longk && w_out == nullptr) return launch_decode_longk(v, x, c, M, s);
  if (resident && w_out == nullptr) return launch_decode_resident(v, x, c, M, s);
  // ... and of its sibling for odd group sizes and ragged K (M <= 64, W4 only)
  const bool general = !resident && !longk && !MX && decode_general_applies(v, x, c, M) &&
                       (w_out == nullptr || ((uintptr_t)w_out & 15) == 0);
  if (general && w_out == nullptr) return launch_decode_general(v, x, c, M, s);
  if (!resident && !general && !longk) {
    if (try_tile_dma(v, x, c, M, s, w_out, &terr)) return terr;
    if (try_tile<MX>(v, x, c, M, s, w_out, &terr)) return terr;
  }
  // Rows of packed words are 16-byte aligned when K % 32 == 0 (one dwordx4 per lane
  // slice); K % 8 == 0 still gives whole words and 16-byte aligned activation rows.
  const bool aligned = (v.K % 8 == 0) && (((uintptr_t)x) & 15) == 0 &&
                       (w_out == nullptr || ((uintptr_t)w_out & 15) == 0);
  if (aligned) {
    // Measured on N = 4096 .. 14336, K = 4096 .. 11008: the K-split kernel wins for
    // M <= 16 unless N is large enough to give the streaming kernel a full grid.
    const bool ksplit = M <= 8 || (M <= 16 && v.N < 8192) || resident || general || longk;
    if (ksplit) {
      if (MX) return launch_decode<2>(v, x, c, M, s, w_out, wvec);
      return v.symmetric ? launch_decode<0>(v, x, c, M, s, w_out, wvec)
                         : launch_decode<1>(v, x, c, M, s, w_out, wvec);
    }
    if (MX) return launch_stream<2>(v, x, c, M, s, w_out, wvec);
    return v.symmetric ? launch_stream<0>(v, x, c, M, s, w_out, wvec)
                       : launch_stream<1>(v, x, c, M, s, w_out, wvec);
  }
  if (M <= 16) return launch_tiles<MX, 1>(v, x, c, M, s, w_out);
  if (M <= 32) return launch_tiles<MX, 2>(v, x, c, M, s, w_out);
  return launch_tiles<MX, 4>(v, x, c, M, s, w_out);
}

hipError_t launch_gemm_mfma(const WView& v, const w4_half* x, w4_half* c, int M,
                            hipStream_t s, w4_half* w_out) {
  return v.mx ? launch_fmt<1>(v, x, c, M, s, w_out) : launch_fmt<0>(v, x, c, M, s, w_out);
}

}  // namespace w4k
