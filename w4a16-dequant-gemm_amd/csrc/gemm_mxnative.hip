// W4A4: c[M,N] = X[M,K] * W[N,K]^T with BOTH operands in packed MXFP4, on the
// gfx950 scaled matrix cores (v_mfma_scale_f32_16x16x128_f8f6f4).
//
// No counterpart in the reference, whose MXFP4 kernels expand the weights to
// FP16 and keep FP16 activations (mxfused.cuh:166-198, 291-307).  Here nothing
// is expanded: a lane's A operand is 32 consecutive E2M1 codes of one row --
// exactly one 16-byte piece of the packed row (mx.hpp:29-41: 8 codes per word,
// low nibble first) -- and its block scale is the row's E8M0 byte for that
// 32-block, applied by the instruction.  Products of E2M1 values and
// power-of-two scales are exact in FP32; the instruction accumulates in FP32.
// The result equals the FP64 product of the two dequantized operands up to FP32
// accumulation and the final FP16 rounding (whenever scale * magnitude is
// representable in FP16, which is what dequant_all_mx returns).
//
// Layout of the instruction (checked on the device against a host product):
//   A: lane l holds row l%16, k-block l/16 (32 codes, 4 dwords)
//   B: lane l holds column l%16, k-block l/16
//   D: lane l holds D[4*(l/16) + i][l%16], i = 0..3
// W supplies A (rows n), X supplies B (columns m): a lane ends with four
// consecutive n of one m.
#include "dq.cuh"
#include "kernels.h"

namespace w4k {
namespace {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));

constexpr int NV_WAVES = 8;   // waves of a decode workgroup (they split K)
constexpr int FMT_FP4 = 4;    // operand format code of the instruction

// One MFMA over 128 k: every lane brings 32 codes and, in byte 0 of its scale
// register, the E8M0 byte of that 32-block.
__device__ __forceinline__ f4 mfma_fp4(u4 a, uint32_t sa, u4 b, uint32_t sb, f4 c) {
  const v4i a4 = __builtin_bit_cast(v4i, a), b4 = __builtin_bit_cast(v4i, b);
  // FP4 operands occupy the low four of the eight operand registers
  const v8i va = __builtin_shufflevector(a4, a4, 0, 1, 2, 3, -1, -1, -1, -1);
  const v8i vb = __builtin_shufflevector(b4, b4, 0, 1, 2, 3, -1, -1, -1, -1);
  return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(va, vb, c, FMT_FP4, FMT_FP4, 0,
                                                          (int)sa, 0, (int)sb);
}

// A lane's share of one 512-k super-step of a packed row: block 4j + g of the
// super-step for j = 0..3 (g = lane / 16), so that load j of the four lane
// groups covers one contiguous 64-byte piece of every row, and MFMA j contracts
// 128 consecutive k.  sc[j] carries the block's scale in byte 0.  FULL: every
// block exists and rows are 16-byte aligned.  Otherwise words past the row read
// as zero codes, codes past K are masked off, and missing blocks take the
// neutral scale byte 127.
template <bool FULL>
__device__ __forceinline__ void load_blocks(const uint32_t* __restrict__ qrow,
                                            const uint8_t* __restrict__ srow, int ss, int g,
                                            int B, int wk, int K, u4 q[4], uint32_t sc[4]) {
  if (FULL) {
#pragma unroll
    for (int j = 0; j < 4; ++j) q[j] = *(const u4*)(qrow + (size_t)(ss * 16 + 4 * j + g) * 4);
    const u4 s16 = *(const u4*)(srow + ss * 16);
#pragma unroll
    for (int j = 0; j < 4; ++j) sc[j] = s16[j] >> (8 * g);
  } else {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int b = ss * 16 + 4 * j + g;
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const int wi = b * 4 + t;
        uint32_t word = wi < wk ? qrow[wi] : 0u;
        if (wi == wk - 1 && (K & 7)) word &= (1u << (4 * (K & 7))) - 1u;
        q[j][t] = word;
      }
      sc[j] = b < B ? srow[b] : 127u;
    }
  }
}

// Skinny M: a workgroup owns 16*NT rows of W and 16*MT rows of X (grid.y walks
// further X rows); its 8 waves take 512-k super-steps round-robin.  A wave
// loads the X pieces of its super-step once and reuses them for the NT row
// tiles, so X crosses L2 -> CU once per workgroup.  Partial sums meet in LDS
// and are added in wave order.
template <int MT, int NT, bool FULL>
__global__ __launch_bounds__(NV_WAVES * 64) void mxn_decode_kernel(
    const uint32_t* __restrict__ wq, const uint8_t* __restrict__ ws,
    const uint32_t* __restrict__ xq, const uint8_t* __restrict__ xs, w4_half* __restrict__ c,
    int N, int K, int B, int M) {
  __shared__ f4 red[NV_WAVES][NT * MT][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int wk = words(K);
  const int n0 = blockIdx.x * (16 * NT), m0 = blockIdx.y * (16 * MT);
  const uint32_t* wrow[NT];
  const uint8_t* wsrow[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    const int n = n0 + nt * 16 + r < N ? n0 + nt * 16 + r : N - 1;
    wrow[nt] = wq + (size_t)n * wk;
    wsrow[nt] = ws + (size_t)n * B;
  }
  const uint32_t* xrow[MT];
  const uint8_t* xsrow[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = m0 + mt * 16 + r < M ? m0 + mt * 16 + r : M - 1;
    xrow[mt] = xq + (size_t)m * wk;
    xsrow[mt] = xs + (size_t)m * B;
  }
  f4 acc[NT][MT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[nt][mt] = f4{0.f, 0.f, 0.f, 0.f};

  const int supers = (B + 15) >> 4;
  for (int ss = wave; ss < supers; ss += NV_WAVES) {
    u4 b[MT][4], a[NT][4];
    uint32_t sb[MT][4], sa[NT][4];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
      load_blocks<FULL>(wrow[nt], wsrow[nt], ss, g, B, wk, K, a[nt], sa[nt]);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
      load_blocks<FULL>(xrow[mt], xsrow[mt], ss, g, B, wk, K, b[mt], sb[mt]);
    // every load of the super-step is in flight before the first product waits
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          acc[nt][mt] = mfma_fp4(a[nt][j], sa[nt][j], b[mt][j], sb[mt][j], acc[nt][mt]);
  }
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) red[wave][nt * MT + mt][lane] = acc[nt][mt];
  __syncthreads();
  // NT * MT * 64 lane slots of four n each
  for (int o = threadIdx.x; o < NT * MT * 64; o += NV_WAVES * 64) {
    const int t = o >> 6, l = o & 63;
    const int nt = t / MT, mt = t - nt * MT;
    f4 sum = red[0][t][l];
#pragma unroll
    for (int w = 1; w < NV_WAVES; ++w) sum += red[w][t][l];
    const int m = m0 + mt * 16 + (l & 15), nn = n0 + nt * 16 + 4 * (l >> 4);
    if (m >= M) continue;
    w4_half* dst = c + (size_t)m * N + nn;
    if (nn + 3 < N && ((uintptr_t)dst & 7) == 0) {
      h4 out;
#pragma unroll
      for (int i = 0; i < 4; ++i) out[i] = (_Float16)sum[i];
      *(h4*)dst = out;
    } else {
      const int left = N - nn;
      if (left > 0) dst[0] = __builtin_bit_cast(uint16_t, (_Float16)sum[0]);
      if (left > 1) dst[1] = __builtin_bit_cast(uint16_t, (_Float16)sum[1]);
      if (left > 2) dst[2] = __builtin_bit_cast(uint16_t, (_Float16)sum[2]);
      if (left > 3) dst[3] = __builtin_bit_cast(uint16_t, (_Float16)sum[3]);
    }
  }
}

template <int MT, int NT>
hipError_t launch_decode_nt(const w4_packed_mx_view& w, const w4_packed_mx_view& x, w4_half* c,
                            hipStream_t s) {
  const int N = w.N, K = w.K, M = x.N;
  const bool full = K % 512 == 0 && ((uintptr_t)w.q & 15) == 0 && ((uintptr_t)x.q & 15) == 0 &&
                    ((uintptr_t)w.scales & 15) == 0 && ((uintptr_t)x.scales & 15) == 0;
  const dim3 grid((unsigned)((N + 16 * NT - 1) / (16 * NT)),
                  (unsigned)((M + 16 * MT - 1) / (16 * MT)));
  const dim3 block(NV_WAVES * 64);
  if (full)
    mxn_decode_kernel<MT, NT, true><<<grid, block, 0, s>>>(w.q, w.scales, x.q, x.scales, c, N,
                                                          K, w.B, M);
  else
    mxn_decode_kernel<MT, NT, false><<<grid, block, 0, s>>>(w.q, w.scales, x.q, x.scales, c, N,
                                                           K, w.B, M);
  return hipGetLastError();
}

// Row tiles per workgroup: as many as keep at least one workgroup per CU.
template <int MT>
hipError_t launch_decode(const w4_packed_mx_view& w, const w4_packed_mx_view& x, w4_half* c,
                         hipStream_t s) {
  const int tiles = (w.N + 15) / 16;
  const int mblocks = (x.N + 16 * MT - 1) / (16 * MT);
  // more row tiles per workgroup cut the X traffic (every workgroup reads all of
  // its X rows through L2): worth it from three X tiles on, while a workgroup per
  // CU remains (N = 14336, M = 64: 21.8 us with three row tiles, 29.5 us with one)
  const int nt = MT >= 3 ? tiles * mblocks / 256 : 1;
  if (nt >= 3) return launch_decode_nt<MT, 3>(w, x, c, s);
  if (nt >= 2) return launch_decode_nt<MT, 2>(w, x, c, s);
  return launch_decode_nt<MT, 1>(w, x, c, s);
}

// ---- large M: LDS-tiled kernel -----------------------------------------------
// Uses the 32x32x64 form of the instruction (measured 8.1 PFLOP/s on FP4 against
// 5.8 for 16x16x128; same lane scheme: A lane l = row l%32, k-block l/32; D lane
// l = column l%32, rows 4*(l/32) + e%4 + 8*(e/4), e = 0..15).
//
// A workgroup of 4 waves (2 x 2) owns 256 rows of W x 128 rows of X; a wave 128 x
// 64 = 4 x 2 MFMA tiles, two MFMAs deep per 128-k step (8 waves of 64 x 64
// measured the same).  Memory is read 256 k at a
// time -- 8 threads take the 128 bytes of a row, so every cache line that crosses
// L2 -> CU is used whole (with 64-byte pieces each line crossed twice and the L2
// bandwidth, not the matrix pipe, set the pace) -- into a ring of TL_PAIRS register
// slots, and goes on to LDS still packed, one 128-k half per step (64 bytes a row,
// rows padded to 80 so that 16 rows x 16 bytes fall on distinct banks); a lane
// reads each operand with one ds_read_b128.  Scale bytes travel the same way, one
// dword (4 blocks) per row and step; a lane shifts its block's byte down.
// Software pipeline, one barrier per step: while the MFMAs of step k run from
// registers, the operands of step k+1 are read from one LDS buffer and step k+2
// is written into the other.
constexpr int TL_TN = 256, TL_TM = 128, TL_ROWS = TL_TN + TL_TM;
constexpr int TL_ROWB = 80;   // LDS bytes per row and step
constexpr int TL_WN = 2;                       // waves along n (and 2 along m)
constexpr int TL_THREADS = 64 * TL_WN * 2;
constexpr int TL_NT = TL_TN / (32 * TL_WN);    // 32-row MFMA tiles of W per wave
constexpr int TL_RP = TL_THREADS / 4;          // rows one pass of the workgroup fetches
constexpr int TL_WI = TL_TN / TL_RP, TL_XI = TL_TM / TL_RP;
constexpr int TL_PAIRS = 2;   // 256-k register slots in flight
constexpr int TL_STAGE = TL_ROWS * TL_ROWB + TL_ROWS * 4;

typedef float f16v __attribute__((ext_vector_type(16)));

__device__ __forceinline__ f16v mfma_fp4_32(u4 a, uint32_t sa, u4 b, uint32_t sb, f16v c) {
  const v4i a4 = __builtin_bit_cast(v4i, a), b4 = __builtin_bit_cast(v4i, b);
  const v8i va = __builtin_shufflevector(a4, a4, 0, 1, 2, 3, -1, -1, -1, -1);
  const v8i vb = __builtin_shufflevector(b4, b4, 0, 1, 2, 3, -1, -1, -1, -1);
  return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(va, vb, c, FMT_FP4, FMT_FP4, 0, (int)sa,
                                                         0, (int)sb);
}

struct TileRegs {  // one thread's share of 256 k on its way to LDS
  u4 w[2][TL_WI], x[2][TL_XI];  // [128-k half][row t/4 + TL_RP i], 16-byte piece t%4
  u2 sw, sx;         // the two steps' scale dwords of W row t%256 / X row t%128
};
struct TileFrags {  // one lane's MFMA operands of a step: [k half][tile]
  u4 a[2][TL_NT], b[2][2];
  uint32_t sa[TL_NT], sb[2];  // the rows' four scale bytes
};

template <int PAIRS>
__global__ __launch_bounds__(TL_THREADS) void mxn_tile_kernel(
    const uint32_t* __restrict__ wq, const uint8_t* __restrict__ ws,
    const uint32_t* __restrict__ xq, const uint8_t* __restrict__ xs, w4_half* __restrict__ c,
    int N, int K, int B, int M, int tiles_n, int tiles_m) {
  __shared__ __attribute__((aligned(16))) uint8_t lds[2][TL_STAGE];
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int r = lane & 31, h = lane >> 5;
  const int wn = wave % TL_WN, wm = wave / TL_WN;  // TL_WN x 2 waves
  // XCD-aware order: consecutive workgroup ids land on different XCDs, so give
  // each XCD a contiguous run of the tile order (m fastest: its workgroups share
  // a few W tiles and walk X)
  int L = blockIdx.x;
  const int total = tiles_n * tiles_m;
  if (total % 8 == 0) L = (L & 7) * (total >> 3) + (L >> 3);
  const int n0 = (L / tiles_m) * TL_TN, m0 = (L % tiles_m) * TL_TM;
  const int wk = K >> 3;  // words per row (K % 256 == 0)

  // byte offsets of this thread's rows (32-bit: tile_applies bounds the operands)
  uint32_t wo[TL_WI], xo[TL_XI];
#pragma unroll
  for (int i = 0; i < TL_WI; ++i) {
    const int n = n0 + (t >> 2) + TL_RP * i;
    wo[i] = ((uint32_t)(n < N ? n : N - 1) * (uint32_t)wk + (t & 3) * 4) * 4u;
  }
#pragma unroll
  for (int i = 0; i < TL_XI; ++i) {
    const int m = m0 + (t >> 2) + TL_RP * i;
    xo[i] = ((uint32_t)(m < M ? m : M - 1) * (uint32_t)wk + (t & 3) * 4) * 4u;
  }
  const uint32_t swo = (uint32_t)(n0 + (t & 255) < N ? n0 + (t & 255) : N - 1) * (uint32_t)B;
  const uint32_t sxo = (uint32_t)(m0 + (t & 127) < M ? m0 + (t & 127) : M - 1) * (uint32_t)B;
  const char* wqb = (const char*)wq;
  const char* xqb = (const char*)xq;

  const int steps = K >> 7, pairs = K >> 8;
  // the two 64-byte halves of a row's line are requested back to back
  auto fetch = [&](TileRegs& q, int p) {
    const uint32_t pp = (uint32_t)(p < pairs ? p : pairs - 1);  // past the end: valid, never used
#pragma unroll
    for (int i = 0; i < TL_WI; ++i) {
      q.w[0][i] = *(const u4*)(wqb + (wo[i] + pp * 128u));
      q.w[1][i] = *(const u4*)(wqb + (wo[i] + pp * 128u + 64u));
    }
#pragma unroll
    for (int i = 0; i < TL_XI; ++i) {
      q.x[0][i] = *(const u4*)(xqb + (xo[i] + pp * 128u));
      q.x[1][i] = *(const u4*)(xqb + (xo[i] + pp * 128u + 64u));
    }
    q.sw = *(const u2*)(ws + (swo + pp * 8u));
    q.sx = *(const u2*)(xs + (sxo + pp * 8u));
  };
  // One 128-k half of a slot goes to LDS.  `keep` is 0 for a step past the end of
  // K: its codes go in as zeros, so the loop needs no branch for a ragged last
  // group of steps.
  auto stage = [&](const TileRegs& q, int buf, int half, uint32_t keep) {
    uint8_t* base = lds[buf];
#pragma unroll
    for (int i = 0; i < TL_WI; ++i)
      *(u4*)(base + ((t >> 2) + TL_RP * i) * TL_ROWB + (t & 3) * 16) = q.w[half][i] & keep;
#pragma unroll
    for (int i = 0; i < TL_XI; ++i)
      *(u4*)(base + (TL_TN + (t >> 2) + TL_RP * i) * TL_ROWB + (t & 3) * 16) = q.x[half][i] & keep;
    uint32_t* sc = (uint32_t*)(base + TL_ROWS * TL_ROWB);
    // several threads hold (and write) the same row's scale dword
    sc[t & 255] = q.sw[half] & keep;
    sc[TL_TN + (t & 127)] = q.sx[half] & keep;
  };
  auto read_frags = [&](TileFrags& f, int buf) {
    const uint8_t* base = lds[buf];
    const uint32_t* sc = (const uint32_t*)(base + TL_ROWS * TL_ROWB);
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int row = TL_TN + wm * 64 + j * 32 + r;
      f.b[0][j] = *(const u4*)(base + row * TL_ROWB + h * 16);
      f.b[1][j] = *(const u4*)(base + row * TL_ROWB + (2 + h) * 16);
      f.sb[j] = sc[row];
    }
#pragma unroll
    for (int i = 0; i < TL_NT; ++i) {
      const int row = wn * (32 * TL_NT) + i * 32 + r;
      f.a[0][i] = *(const u4*)(base + row * TL_ROWB + h * 16);
      f.a[1][i] = *(const u4*)(base + row * TL_ROWB + (2 + h) * 16);
      f.sa[i] = sc[row];
    }
  };

  f16v acc[TL_NT][2];
#pragma unroll
  for (int i = 0; i < TL_NT; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  auto multiply = [&](const TileFrags& f) {
#pragma unroll
    for (int kh = 0; kh < 2; ++kh) {
      const int sh = 16 * kh + 8 * h;  // this lane's block of the step: 2 kh + h
#pragma unroll
      for (int i = 0; i < TL_NT; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          acc[i][j] = mfma_fp4_32(f.a[kh][i], f.sa[i] >> sh, f.b[kh][j], f.sb[j] >> sh, acc[i][j]);
    }
  };

  TileRegs ring[PAIRS];
  TileFrags frags[2];
  // steps 2p and 2p+1 travel in ring slot p % PAIRS
#pragma unroll
  for (int d = 0; d < PAIRS; ++d) fetch(ring[d], d);
  stage(ring[0], 0, 0, ~0u);
  stage(ring[0], 1, 1, ~0u);
  fetch(ring[0], PAIRS);
  __syncthreads();
  read_frags(frags[0], 0);
  __syncthreads();  // buffer 0 is rewritten in the first iteration

  // The unrolled body spans PAIRS slots = 2 * PAIRS steps: slot, half and buffer
  // parity are constants, and there is no branch (every wait counts exactly the
  // loads it needs).
#pragma unroll 1
  for (int kb = 0; kb < steps; kb += 2 * PAIRS) {
#pragma unroll
    for (int u = 0; u < 2 * PAIRS; ++u) {
      const int k = kb + u;
      const int slot = ((u + 2) >> 1) % PAIRS;  // of step k + 2
      read_frags(frags[(u + 1) & 1], (u + 1) & 1);
      stage(ring[slot], u & 1, u & 1, k + 2 < steps ? ~0u : 0u);
      if (u & 1) fetch(ring[slot], ((k + 2) >> 1) + PAIRS);
      multiply(frags[u & 1]);
      __syncthreads();
    }
  }

  // lane: m = .. + r; e = 4 q + p holds n = .. + 8 q + 4 h + p
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int m = m0 + wm * 64 + j * 32 + r;
    if (m >= M) continue;
#pragma unroll
    for (int i = 0; i < TL_NT; ++i)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int nn = n0 + wn * (32 * TL_NT) + i * 32 + 8 * q + 4 * h;
        w4_half* dst = c + (size_t)m * N + nn;
        if (nn + 3 < N && ((uintptr_t)dst & 7) == 0) {
          h4 out;
#pragma unroll
          for (int e = 0; e < 4; ++e) out[e] = (_Float16)acc[i][j][4 * q + e];
          *(h4*)dst = out;
        } else {
          const int left = N - nn;
          if (left > 0) dst[0] = __builtin_bit_cast(uint16_t, (_Float16)acc[i][j][4 * q + 0]);
          if (left > 1) dst[1] = __builtin_bit_cast(uint16_t, (_Float16)acc[i][j][4 * q + 1]);
          if (left > 2) dst[2] = __builtin_bit_cast(uint16_t, (_Float16)acc[i][j][4 * q + 2]);
          if (left > 3) dst[3] = __builtin_bit_cast(uint16_t, (_Float16)acc[i][j][4 * q + 3]);
        }
      }
  }
}

bool tile_applies(const w4_packed_mx_view& w, const w4_packed_mx_view& x) {
  // below a few hundred rows of X the skinny kernel's grid.y walk is faster (measured:
  // M = 256 at N = 4096 takes 21 us there, 37 us here on 32 workgroups)
  return x.N >= 384 && w.K % 256 == 0 && (long long)w.N * w.K < (1LL << 32) &&
         (long long)x.N * x.K < (1LL << 32) && ((uintptr_t)w.q & 15) == 0 && ((uintptr_t)x.q & 15) == 0 &&
         ((uintptr_t)w.scales & 7) == 0 && ((uintptr_t)x.scales & 7) == 0;
}

hipError_t launch_tile(const w4_packed_mx_view& w, const w4_packed_mx_view& x, w4_half* c,
                       hipStream_t s) {
  const int tiles_n = (w.N + TL_TN - 1) / TL_TN, tiles_m = (x.N + TL_TM - 1) / TL_TM;
  if ((long long)tiles_n * tiles_m > 0x7FFFFFFFLL) return hipErrorInvalidConfiguration;
  mxn_tile_kernel<TL_PAIRS><<<dim3((unsigned)(tiles_n * tiles_m)), dim3(TL_THREADS), 0, s>>>(
      w.q, w.scales, x.q, x.scales, c, w.N, w.K, w.B, x.N, tiles_n, tiles_m);
  return hipGetLastError();
}

}  // namespace

hipError_t launch_gemm_mx_w4a4(const w4_packed_mx_view& w, const w4_packed_mx_view& x,
                               w4_half* c, hipStream_t s) {
  const int M = x.N;
  if (tile_applies(w, x)) return launch_tile(w, x, c, s);
  if (M <= 16) return launch_decode<1>(w, x, c, s);
  if (M <= 32) return launch_decode<2>(w, x, c, s);
  if (M <= 48) return launch_decode<3>(w, x, c, s);
  return launch_decode<4>(w, x, c, s);
}

}  // namespace w4k
