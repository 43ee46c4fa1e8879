// W4A4 / W4A8: c[M,N] = X[M,K] * W[N,K]^T with packed MXFP4 weights against
// activations that are block-scaled too -- packed MXFP4, or E4M3 bytes under the
// same E8M0 block scales -- on the gfx950 scaled matrix cores
// (v_mfma_scale_f32_{16x16x128,32x32x64}_f8f6f4).
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
//   B: lane l holds column l%16, k-block l/16 (4-bit; an 8-bit B differs, see
//      load_blocks8)
//   D: lane l holds D[4*(l/16) + i][l%16], i = 0..3
// W supplies A (rows n), X supplies B (columns m): a lane ends with four
// consecutive n of one m.
#include <atomic>

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

// The same with E4M3 activations: the B operand is 32 bytes (all eight registers).
constexpr int FMT_FP8 = 0;
__device__ __forceinline__ f4 mfma_fp4_fp8(u4 a, uint32_t sa, u4 b0, u4 b1, uint32_t sb, f4 c) {
  const v4i a4 = __builtin_bit_cast(v4i, a);
  const v8i va = __builtin_shufflevector(a4, a4, 0, 1, 2, 3, -1, -1, -1, -1);
  const v4i lo = __builtin_bit_cast(v4i, b0), hi = __builtin_bit_cast(v4i, b1);
  const v8i vb = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(va, vb, c, FMT_FP4, FMT_FP8, 0,
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

// The matching share of a row of E4M3 bytes (K a multiple of 32).  An 8-bit
// operand is laid out differently from a 4-bit one (checked on the device element
// by element): of the 128 k of MFMA j, lane group g holds k 16g..16g+15 in its
// first four registers and k 64+16g..64+16g+15 in the other four, while its scale
// register still carries the scale of 32-block g of those 128 k.  The four lane
// groups of either load cover 64 contiguous bytes of every row.
template <bool FULL>
__device__ __forceinline__ void load_blocks8(const uint8_t* __restrict__ qrow,
                                             const uint8_t* __restrict__ srow, int ss, int g,
                                             int B, int K, u4 q[4][2], uint32_t sc[4]) {
  if (FULL) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint8_t* p = qrow + (size_t)ss * 512 + 128 * j + 16 * g;
      q[j][0] = *(const u4*)p;
      q[j][1] = *(const u4*)(p + 64);
    }
    const u4 s16 = *(const u4*)(srow + ss * 16);
#pragma unroll
    for (int j = 0; j < 4; ++j) sc[j] = s16[j] >> (8 * g);
  } else {
    const u4 zero = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int k = ss * 512 + 128 * j + 16 * g, b = ss * 16 + 4 * j + g;
      q[j][0] = k < K ? *(const u4*)(qrow + k) : zero;
      q[j][1] = k + 64 < K ? *(const u4*)(qrow + k + 64) : zero;
      sc[j] = b < B ? srow[b] : 127u;
    }
  }
}

// Skinny M: a workgroup owns 16*NT rows of W and 16*MT rows of X (grid.y walks
// further X rows); its 8 waves take 512-k super-steps round-robin.  A wave
// loads the X pieces of its super-step once and reuses them for the NT row
// tiles, so X crosses L2 -> CU once per workgroup.  Partial sums meet in LDS
// and are added in wave order.
// XF8: X holds E4M3 bytes (K per row) instead of packed E2M1 codes.
template <int MT, int NT, bool FULL, bool XF8>
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
    xrow[mt] = xq + (size_t)m * (XF8 ? K >> 2 : wk);  // K bytes or words(K) words a row
    xsrow[mt] = xs + (size_t)m * B;
  }
  f4 acc[NT][MT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[nt][mt] = f4{0.f, 0.f, 0.f, 0.f};

  const int supers = (B + 15) >> 4;
  for (int ss = wave; ss < supers; ss += NV_WAVES) {
    u4 b[MT][4][XF8 ? 2 : 1], a[NT][4];
    uint32_t sb[MT][4], sa[NT][4];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
      load_blocks<FULL>(wrow[nt], wsrow[nt], ss, g, B, wk, K, a[nt], sa[nt]);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      if constexpr (XF8) {
        load_blocks8<FULL>((const uint8_t*)xrow[mt], xsrow[mt], ss, g, B, K, b[mt], sb[mt]);
      } else {
        u4 q[4];
        load_blocks<FULL>(xrow[mt], xsrow[mt], ss, g, B, wk, K, q, sb[mt]);
#pragma unroll
        for (int j = 0; j < 4; ++j) b[mt][j][0] = q[j];
      }
    }
    // every load of the super-step is in flight before the first product waits
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          if constexpr (XF8)
            acc[nt][mt] = mfma_fp4_fp8(a[nt][j], sa[nt][j], b[mt][j][0], b[mt][j][1], sb[mt][j],
                                       acc[nt][mt]);
          else
            acc[nt][mt] = mfma_fp4(a[nt][j], sa[nt][j], b[mt][j][0], sb[mt][j], acc[nt][mt]);
        }
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

// FULL_ONLY: the caller has checked K % 512 == 0 and the guarded form of this shape is
// not compiled (it does not fit the register file); unaligned operands then take two
// row tiles.
template <int MT, int NT, bool XF8, bool FULL_ONLY = false>
hipError_t launch_decode_nt(const w4_packed_mx_view& w, const void* xq, const uint8_t* xs, int M,
                            w4_half* c, hipStream_t s) {
  const int N = w.N, K = w.K;
  const bool full = K % 512 == 0 && ((uintptr_t)w.q & 15) == 0 && ((uintptr_t)xq & 15) == 0 &&
                    ((uintptr_t)w.scales & 15) == 0 && ((uintptr_t)xs & 15) == 0;
  const dim3 grid((unsigned)((N + 16 * NT - 1) / (16 * NT)),
                  (unsigned)((M + 16 * MT - 1) / (16 * MT)));
  const dim3 block(NV_WAVES * 64);
  if (full) {
    mxn_decode_kernel<MT, NT, true, XF8><<<grid, block, 0, s>>>(
        w.q, w.scales, (const uint32_t*)xq, xs, c, N, K, w.B, M);
  } else if constexpr (FULL_ONLY) {
    return launch_decode_nt<MT, 2, XF8>(w, xq, xs, M, c, s);
  } else {
    mxn_decode_kernel<MT, NT, false, XF8><<<grid, block, 0, s>>>(
        w.q, w.scales, (const uint32_t*)xq, xs, c, N, K, w.B, M);
  }
  return hipGetLastError();
}

// Row tiles per workgroup: as many as keep at least one workgroup per CU.
template <int MT, bool XF8>
hipError_t launch_decode(const w4_packed_mx_view& w, const void* xq, const uint8_t* xs, int M,
                         w4_half* c, hipStream_t s) {
  const int tiles = (w.N + 15) / 16;
  const int mblocks = (M + 16 * MT - 1) / (16 * MT);
  // more row tiles per workgroup cut the X traffic (every workgroup reads all of
  // its X rows through L2): worth it from three X tiles on, while a workgroup per
  // CU remains (N = 14336, M = 64: 21.8 us with three row tiles, 29.5 us with one)
  const int nt = (MT >= 3 || (XF8 && MT == 2)) ? tiles * mblocks / 256 : 1;
  // Four X tiles times three row tiles do not fit the register file (that instantiation
  // spilled 37 - 85 VGPRs: N = 14336, M = 64, 22.2 / 42.7 us with MXFP4 / MXFP8 activations
  // against 18.3 / 27.1 with two row tiles), nor do three times three with 8-bit X on a
  // ragged K; 8-bit X never runs four X tiles (launch_skinny).  None of those is compiled.
  if constexpr (MT < 4) {
    if (nt >= 3) {
      constexpr bool fits_ragged = !(XF8 && MT == 3);
      const bool full = w.K % 512 == 0;
      if (fits_ragged || full) return launch_decode_nt<MT, 3, XF8, !fits_ragged>(w, xq, xs, M, c, s);
    }
  }
  if (nt >= 2) return launch_decode_nt<MT, 2, XF8>(w, xq, xs, M, c, s);
  return launch_decode_nt<MT, 1, XF8>(w, xq, xs, M, c, s);
}

template <bool XF8>
hipError_t launch_skinny(const w4_packed_mx_view& w, const void* xq, const uint8_t* xs, int M,
                         w4_half* c, hipStream_t s) {
  if (M <= 16) return launch_decode<1, XF8>(w, xq, xs, M, c, s);
  if (M <= 32) return launch_decode<2, XF8>(w, xq, xs, M, c, s);
  if (M <= 48) return launch_decode<3, XF8>(w, xq, xs, M, c, s);
  // 8-bit X: four X tiles hold twice the operand registers of 4-bit ones and spill even
  // with two row tiles; 49 .. 64 rows go in two passes of 32 (grid.y)
  if constexpr (XF8) return launch_decode<2, XF8>(w, xq, xs, M, c, s);
  else return launch_decode<4, XF8>(w, xq, xs, M, c, s);
}

// ---- large M: LDS-tiled kernel -----------------------------------------------
// Uses the 32x32x64 form of the instruction (measured 7.9 PFLOP/s on FP4 against
// 5.8 for 16x16x128; same lane scheme: A lane l = row l%32, k-block l/32; D lane
// l = column l%32, rows 4*(l/32) + e%4 + 8*(e/4), e = 0..15).  A workgroup owns
// 256 rows of W x 128 rows of X.
constexpr int TL_TN = 256, TL_TM = 128, TL_ROWS = TL_TN + TL_TM;

typedef float f16v __attribute__((ext_vector_type(16)));

__device__ __forceinline__ f16v mfma_fp4_32(u4 a, uint32_t sa, u4 b, uint32_t sb, f16v c) {
  const v4i a4 = __builtin_bit_cast(v4i, a), b4 = __builtin_bit_cast(v4i, b);
  const v8i va = __builtin_shufflevector(a4, a4, 0, 1, 2, 3, -1, -1, -1, -1);
  const v8i vb = __builtin_shufflevector(b4, b4, 0, 1, 2, 3, -1, -1, -1, -1);
  return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(va, vb, c, FMT_FP4, FMT_FP4, 0, (int)sa,
                                                         0, (int)sb);
}

// Operands go global -> LDS directly.
// global_load_lds_dwordx4 writes lane l's 16 bytes to LDS at (wave-uniform base)
// + 16 l, so a wave instruction fills 1 KB, and which piece of which row a lane
// fetches is free to choose.  A stage holds 256 k: 128 bytes = one cache line per
// row, so every line crosses L2 -> CU once, whole.  An instruction takes 8 rows;
// lane l fetches row l/8, piece (l%8) ^ key(row), key(R) = (R/2) % 8: eight
// neighbouring lanes still cover one contiguous line (coalesced), and the 16
// rows x 16 bytes a lane group reads back for one MFMA operand land on 16
// distinct 16-byte bank groups (conflict-free ds_read_b128 without padding).
// No staging registers, no ds_write instructions: three stages of 256 k sit in
// LDS (dynamic LDS, 153 KB; two stages, 134 KB, with 8-bit X); one barrier per stage.  Per stage d: multiply
// the first 128 k of d while reading the operands of the second; wait for d+1,
// barrier -- every wave is now done with d's buffer, so request d+3 into it;
// multiply the second 128 k while reading the first operands of d+1.
// XF8: X holds E4M3 bytes -- rows of 256 bytes per stage, four rows per load
// instruction, piece key = row % 16, and room for two stages instead of three.
constexpr int DM_W_BYTES = TL_TN * 128;
constexpr int DM_WN = 4;                                     // waves along n (2 along m)
constexpr int DM_WAVES = 2 * DM_WN;
constexpr int DM_THREADS = 64 * DM_WAVES;
constexpr int DM_NT = TL_TN / (32 * DM_WN);                  // 32-row tiles of W per wave
constexpr int DM_WI = 32 / DM_WAVES;                         // 8-row blocks of W a wave fetches
template <bool XF8>
struct Dm {
  static constexpr int STAGES = XF8 ? 2 : 3;
  static constexpr int X_ROWB = XF8 ? 256 : 128;             // bytes of an X row per stage
  static constexpr int X_BYTES = TL_TM * X_ROWB;
  static constexpr int TILE_BYTES = DM_W_BYTES + X_BYTES;    // 48 / 64 KB, unpadded
  static constexpr int STAGE = TILE_BYTES + 2 * TL_ROWS * 4; // + two scale dwords per row
  static constexpr int XI = X_BYTES / 1024 / DM_WAVES;       // 1 KB blocks of X a wave fetches
  static constexpr int LOADS = DM_WI + XI + 2;               // wave instructions per stage
  static constexpr int NB = XF8 ? 2 : 1;                     // register quads of a B operand
};

template <bool XF8>
struct DmFrags {  // one lane's MFMA operands of a 128-k half: [k half][tile]
  u4 a[2][DM_NT], b[2][2][Dm<XF8>::NB];
  uint32_t sa[DM_NT], sb[2];
};

__device__ __forceinline__ f16v mfma_fp4_fp8_32(u4 a, uint32_t sa, u4 b0, u4 b1, uint32_t sb,
                                                f16v c) {
  const v4i a4 = __builtin_bit_cast(v4i, a);
  const v8i va = __builtin_shufflevector(a4, a4, 0, 1, 2, 3, -1, -1, -1, -1);
  const v4i lo = __builtin_bit_cast(v4i, b0), hi = __builtin_bit_cast(v4i, b1);
  const v8i vb = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(va, vb, c, FMT_FP4, FMT_FP8, 0, (int)sa,
                                                         0, (int)sb);
}

typedef __attribute__((address_space(3))) void* lds_ptr;

// s_waitcnt vmcnt(N) alone (gfx9 encoding: vmcnt in [3:0] and [15:14])
constexpr int waitcnt_vm(int n) { return (n & 0xF) | ((n >> 4) << 14) | 0x0F70; }

extern __shared__ __attribute__((aligned(16))) uint8_t dm_lds[];

template <bool XF8>
__global__ __launch_bounds__(DM_THREADS) void mxn_tile_dma_kernel(
    const uint32_t* __restrict__ wq, const uint8_t* __restrict__ ws,
    const uint32_t* __restrict__ xq, const uint8_t* __restrict__ xs, w4_half* __restrict__ c,
    int N, int K, int B, int M, int tiles_n, int tiles_m) {
  const int t = threadIdx.x, lane = t & 63;
  const int wave = __builtin_amdgcn_readfirstlane(t >> 6);  // in an SGPR: LDS addresses go to M0
  const int r = lane & 31, h = lane >> 5;
  const int wn = wave % DM_WN, wm = wave / DM_WN;  // DM_WN x 2 waves
  // XCD-aware order: consecutive workgroup ids land on different XCDs (each with
  // its own L2), so give each XCD a contiguous run of the tile order, m fastest:
  // its workgroups share a few W tiles and walk X.  (Blocks of 4 x 8 tiles per
  // XCD measured no better.)
  int L = blockIdx.x;
  const int total = tiles_n * tiles_m;
  if (total % 8 == 0) L = (L & 7) * (total >> 3) + (L >> 3);
  const int n0 = (L / tiles_m) * TL_TN, m0 = (L % tiles_m) * TL_TM;
  const int wk = K >> 3;

  // what this lane fetches: row l/8 of an 8-row block, swizzled 16-byte piece.
  // Wave w takes blocks w + 4 i; the key only needs the row's position in its
  // 16-row group: ((block & 1) * 8 + l/8) / 2.
  typedef Dm<XF8> C;
  const int row8 = lane >> 3;
  uint32_t wo[DM_WI], xo[C::XI];  // byte offsets (32-bit: tile_applies bounds the operands)
#pragma unroll
  for (int i = 0; i < DM_WI; ++i) {
    const int blk = wave + DM_WAVES * i, R = blk * 8 + row8, n = n0 + R;
    wo[i] = ((uint32_t)(n < N ? n : N - 1) * (uint32_t)wk) * 4u + (((lane & 7) ^ ((R >> 1) & 7)) * 16);
  }
#pragma unroll
  for (int i = 0; i < C::XI; ++i) {
    const int blk = wave + DM_WAVES * i;
    if (XF8) {  // 4 rows of 256 bytes per instruction, piece key R % 16, K bytes a row
      const int R = blk * 4 + (lane >> 4), m = m0 + R;
      xo[i] = (uint32_t)(m < M ? m : M - 1) * (uint32_t)K + (((lane & 15) ^ (R & 15)) * 16);
    } else {
      const int R = blk * 8 + row8, m = m0 + R;
      xo[i] = ((uint32_t)(m < M ? m : M - 1) * (uint32_t)wk) * 4u +
              (((lane & 7) ^ ((R >> 1) & 7)) * 16);
    }
  }
  // scale dwords: waves 0-3 take W rows 64 wave + lane, the others X rows 64 (wave & 1)
  // + lane (a wave fetches two per stage either way)
  const bool w_scales = wave < 4;
  const int srow = w_scales ? n0 + wave * 64 + lane : m0 + (wave & 1) * 64 + lane;
  const int slim = w_scales ? N : M;
  const uint32_t sco = (uint32_t)(srow < slim ? srow : slim - 1) * (uint32_t)B;
  const uint8_t* scb = w_scales ? ws : xs;
  const uint32_t sc_lds = w_scales ? wave * 256 : TL_TN * 4 + (wave & 1) * 256;
  const char* wqb = (const char*)wq;
  const char* xqb = (const char*)xq;

  const int stages = K >> 8;
  // The loads are written as asm so that the compiler neither tracks them (it would
  // wait for all of them before any LDS read) nor moves LDS reads across them; the
  // vmcnt waits below are by hand.  M0 carries the wave-uniform LDS address.
  auto dma16 = [](const void* gbase, uint32_t goff, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1"
                 :
                 : "v"(goff), "s"(gbase), "s"(lds_addr)
                 : "memory", "m0");
  };
  auto dma4 = [](const void* gbase, uint32_t goff, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dword %0, %1"
                 :
                 : "v"(goff), "s"(gbase), "s"(lds_addr)
                 : "memory", "m0");
  };
  const uint32_t lds0 = (uint32_t)(uintptr_t)(lds_ptr)dm_lds;
  auto request = [&](int d) {
    const uint32_t dd = (uint32_t)(d < stages ? d : stages - 1);  // past the end: valid, never used
    const uint32_t st = lds0 + (uint32_t)(d % C::STAGES) * C::STAGE;
#pragma unroll
    for (int i = 0; i < DM_WI; ++i)
      dma16(wqb, wo[i] + dd * 128u, st + (wave + DM_WAVES * i) * 1024);
#pragma unroll
    for (int i = 0; i < C::XI; ++i)
      dma16(xqb, xo[i] + dd * (uint32_t)C::X_ROWB, st + DM_W_BYTES + (wave + DM_WAVES * i) * 1024);
#pragma unroll
    for (int s2 = 0; s2 < 2; ++s2)  // the two 128-k halves' scale dwords
      dma4(scb, sco + dd * 8u + s2 * 4u, st + C::TILE_BYTES + s2 * (TL_ROWS * 4) + sc_lds);
  };
  // row R of an operand tile, 16-byte piece p (0..7) of the 256 k -> byte offset
  auto at = [](int R, int p) { return (R >> 3) * 1024 + ((R & 7) * 8 + (p ^ ((R >> 1) & 7))) * 16; };
  // operands of the 128-k half s2 of stage d
  // the same for a 256-byte row of E4M3 bytes, piece p in 0..15
  auto at8 = [](int R, int p) { return (R >> 2) * 1024 + ((R & 3) * 16 + (p ^ (R & 15))) * 16; };
  auto read_frags = [&](DmFrags<XF8>& f, int d, int s2) {
    const uint8_t* base = dm_lds + (d % C::STAGES) * C::STAGE;
    const uint32_t* sc = (const uint32_t*)(base + C::TILE_BYTES) + s2 * TL_ROWS;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int row = wm * 64 + j * 32 + r;
#pragma unroll
      for (int kh = 0; kh < 2; ++kh) {
        if constexpr (XF8) {
          // of the 64 k of MFMA kh an 8-bit lane group h holds k 16h.. and 32+16h..
          f.b[kh][j][0] = *(const u4*)(base + DM_W_BYTES + at8(row, 8 * s2 + 4 * kh + h));
          f.b[kh][j][1] = *(const u4*)(base + DM_W_BYTES + at8(row, 8 * s2 + 4 * kh + 2 + h));
        } else {
          f.b[kh][j][0] = *(const u4*)(base + DM_W_BYTES + at(row, 4 * s2 + 2 * kh + h));
        }
      }
      f.sb[j] = sc[TL_TN + row];
    }
#pragma unroll
    for (int i = 0; i < DM_NT; ++i) {
      const int row = wn * (32 * DM_NT) + i * 32 + r;
      f.a[0][i] = *(const u4*)(base + at(row, 4 * s2 + h));
      f.a[1][i] = *(const u4*)(base + at(row, 4 * s2 + 2 + h));
      f.sa[i] = sc[row];
    }
  };

  f16v acc[DM_NT][2];
#pragma unroll
  for (int i = 0; i < DM_NT; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
  auto multiply = [&](const DmFrags<XF8>& f) {
#pragma unroll
    for (int kh = 0; kh < 2; ++kh) {
      const int sh = 16 * kh + 8 * h;
#pragma unroll
      for (int i = 0; i < DM_NT; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
        {
          if constexpr (XF8)
            acc[i][j] = mfma_fp4_fp8_32(f.a[kh][i], f.sa[i] >> sh, f.b[kh][j][0], f.b[kh][j][1],
                                        f.sb[j] >> sh, acc[i][j]);
          else
            acc[i][j] = mfma_fp4_32(f.a[kh][i], f.sa[i] >> sh, f.b[kh][j][0], f.sb[j] >> sh, acc[i][j]);
        }
    }
  };

  DmFrags<XF8> fa, fb;
#pragma unroll
  for (int d = 0; d < C::STAGES; ++d) request(d);
  // stage 0 has landed (this wave's part)
  __builtin_amdgcn_s_waitcnt(waitcnt_vm((C::STAGES - 1) * C::LOADS));
  __syncthreads();
  read_frags(fa, 0, 0);
#pragma unroll 1
  for (int d = 0; d < stages; ++d) {
    read_frags(fb, d, 1);
    __builtin_amdgcn_sched_barrier(0);
    multiply(fa);
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_waitcnt(waitcnt_vm((C::STAGES - 2) * C::LOADS));  // stage d + 1 has landed
    __syncthreads();
    // every wave has read both halves of stage d: its buffer takes the next stage to request
    request(d + C::STAGES);
    read_frags(fa, d + 1, 0);
    __builtin_amdgcn_sched_barrier(0);
    multiply(fb);
    __builtin_amdgcn_sched_barrier(0);
  }
  __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));  // nothing may still be writing LDS at exit

  // A lane holds, of each 32 x 32 tile, n = 8 q + 4 h + e for m = tile row r.  Whole
  // tiles go through LDS (free by now) so that every store instruction writes eight
  // whole 128-byte lines instead of 16 bytes of each of 32: a wave lays its 64 (m)
  // x 64 (n) block out in rows of 144 bytes and reads it back 16 bytes a lane.
  const bool whole = m0 + TL_TM <= M && n0 + TL_TN <= N && (N & 7) == 0 && ((uintptr_t)c & 15) == 0;
  if (whole) {
    constexpr int PITCH = 144;
    __syncthreads();  // no wave reads a stage buffer any more, no load is landing in one
    uint8_t* mine = dm_lds + wave * (64 * PITCH);
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int i = 0; i < DM_NT; ++i)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          h4 out;
#pragma unroll
          for (int e = 0; e < 4; ++e) out[e] = (_Float16)acc[i][j][4 * q + e];
          *(h4*)(mine + (j * 32 + r) * PITCH + i * 64 + q * 16 + h * 8) = out;
        }
    w4_half* cw = c + (size_t)(m0 + wm * 64) * N + n0 + wn * (32 * DM_NT);
#pragma unroll
    for (int it = 0; it < 8; ++it) {
      const int row = it * 8 + (lane >> 3), piece = lane & 7;
      const u4 v = *(const u4*)(mine + row * PITCH + piece * 16);
      *(u4*)(cw + (size_t)row * N + piece * 8) = v;
    }
    return;
  }
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int m = m0 + wm * 64 + j * 32 + r;
    if (m >= M) continue;
#pragma unroll
    for (int i = 0; i < DM_NT; ++i)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int nn = n0 + wn * (32 * DM_NT) + i * 32 + 8 * q + 4 * h;
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

// The same tile for packed-MXFP4 activations with one wave per SIMD: 4 waves, each
// 64 rows of W x all 128 rows of X (2 x 4 tiles of 32x32x64).  A stage (256 k) is
// four steps of 64 k; during the eight MFMAs of a step the wave reads the next
// step's six operands from LDS, and the fifteen load instructions of a stage are
// issued four per step instead of in a row (a wave has one instruction stream to
// keep its SIMD's matrix pipe fed).  Stage d + 2 is requested from the last step of
// stage d - 1, when the barrier there has freed its buffer.
constexpr int D4_WAVES = 4, D4_THREADS = 64 * D4_WAVES;
constexpr int D4_TILE = DM_W_BYTES + TL_TM * 128;           // 48 KB
constexpr int D4_STAGE = D4_TILE + 2 * TL_ROWS * 4;         // + two scale dwords per row
constexpr int D4_STAGES = 3;
constexpr int D4_WI = DM_W_BYTES / 1024 / D4_WAVES;         // 8
constexpr int D4_XI = TL_TM * 128 / 1024 / D4_WAVES;        // 4
constexpr int D4_LOADS = D4_WI + D4_XI + 3;                 // + two dwords of W scales, one of X scales

__global__ __launch_bounds__(D4_THREADS) void mxn_tile4_kernel(
    const uint32_t* __restrict__ wq, const uint8_t* __restrict__ ws,
    const uint32_t* __restrict__ xq, const uint8_t* __restrict__ xs, w4_half* __restrict__ c,
    int N, int K, int B, int M, int tiles_n, int tiles_m) {
  const int t = threadIdx.x, lane = t & 63;
  const int wave = __builtin_amdgcn_readfirstlane(t >> 6);  // in an SGPR: LDS addresses go to M0
  const int r = lane & 31, h = lane >> 5;
  int L = blockIdx.x;
  const int total = tiles_n * tiles_m;
  if (total % 8 == 0) L = (L & 7) * (total >> 3) + (L >> 3);  // a run of the tile order per XCD
  const int n0 = (L / tiles_m) * TL_TN, m0 = (L % tiles_m) * TL_TM;
  const int wk = K >> 3;

  // what this lane fetches: row l/8 of an 8-row block, swizzled 16-byte piece
  const int row8 = lane >> 3;
  uint32_t wo[D4_WI], xo[D4_XI];
#pragma unroll
  for (int i = 0; i < D4_WI; ++i) {
    const int R = (wave + D4_WAVES * i) * 8 + row8, n = n0 + R;
    wo[i] = ((uint32_t)(n < N ? n : N - 1) * (uint32_t)wk) * 4u + (((lane & 7) ^ ((R >> 1) & 7)) * 16);
  }
#pragma unroll
  for (int i = 0; i < D4_XI; ++i) {
    const int R = (wave + D4_WAVES * i) * 8 + row8, m = m0 + R;
    xo[i] = ((uint32_t)(m < M ? m : M - 1) * (uint32_t)wk) * 4u + (((lane & 7) ^ ((R >> 1) & 7)) * 16);
  }
  // scale dwords: W rows 64 wave + lane, both 128-k halves; X rows 64 (wave & 1) + lane, half wave / 2
  const int swrow = n0 + wave * 64 + lane, sxrow = m0 + (wave & 1) * 64 + lane;
  const uint32_t swo = (uint32_t)(swrow < N ? swrow : N - 1) * (uint32_t)B;
  const uint32_t sxo = (uint32_t)(sxrow < M ? sxrow : M - 1) * (uint32_t)B + (uint32_t)(wave >> 1) * 4u;
  const char* wqb = (const char*)wq;
  const char* xqb = (const char*)xq;
  const int stages = K >> 8;
  auto dma16 = [](const void* gbase, uint32_t goff, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1"
                 :
                 : "v"(goff), "s"(gbase), "s"(lds_addr)
                 : "memory", "m0");
  };
  auto dma4 = [](const void* gbase, uint32_t goff, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dword %0, %1"
                 :
                 : "v"(goff), "s"(gbase), "s"(lds_addr)
                 : "memory", "m0");
  };
  const uint32_t lds0 = (uint32_t)(uintptr_t)(lds_ptr)dm_lds;
  auto request_part = [&](int d, uint32_t buf, int part) {  // buf: byte offset of the stage's buffer
    const uint32_t dd = (uint32_t)(d < stages ? d : stages - 1);  // past the end: valid, never used
    const uint32_t st = lds0 + buf;
    if (part < D4_WI) {
      dma16(wqb + dd * 128u, wo[part], st + (wave + D4_WAVES * part) * 1024);
    } else if (part < D4_WI + D4_XI) {
      const int i = part - D4_WI;
      dma16(xqb + dd * 128u, xo[i], st + DM_W_BYTES + (wave + D4_WAVES * i) * 1024);
    } else if (part < D4_WI + D4_XI + 2) {
      const int s2 = part - D4_WI - D4_XI;
      dma4(ws + dd * 8u + s2 * 4u, swo, st + D4_TILE + s2 * (TL_ROWS * 4) + wave * 256);
    } else {
      dma4(xs + dd * 8u, sxo, st + D4_TILE + (wave >> 1) * (TL_ROWS * 4) + TL_TN * 4 + (wave & 1) * 256);
    }
  };
  auto request = [&](int d, uint32_t buf) {
#pragma unroll
    for (int part = 0; part < D4_LOADS; ++part) request_part(d, buf, part);
  };

  // where this lane reads inside a stage buffer: piece 2 u + h of its row in W tile
  // 0 and X tile 0 (the next tile is 4 KB further), its rows' scale dwords
  auto at = [](int R, int p) { return (R >> 3) * 1024 + ((R & 7) * 8 + (p ^ ((R >> 1) & 7))) * 16; };
  uint32_t woff[4], xoff[4];
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    woff[u] = at(wave * 64 + r, 2 * u + h);
    xoff[u] = DM_W_BYTES + at(r, 2 * u + h);
  }
  const uint32_t saoff = D4_TILE + (wave * 64 + r) * 4, sboff = D4_TILE + (TL_TN + r) * 4;

  u4 wv[2][2], xv[2][4];          // operands of the step in hand and of the next
  uint32_t sa[2][2], sb[2][4];    // scale dwords of the 128-k half in hand and of the next
  auto read_ops = [&](int slot, uint32_t buf, int u) {
    const uint8_t* pw = dm_lds + (buf + woff[u]);
    const uint8_t* px = dm_lds + (buf + xoff[u]);
#pragma unroll
    for (int i = 0; i < 2; ++i) wv[slot][i] = *(const u4*)(pw + i * 4096);
#pragma unroll
    for (int j = 0; j < 4; ++j) xv[slot][j] = *(const u4*)(px + j * 4096);
  };
  auto read_scales = [&](int slot, uint32_t buf, int s2) {
    const uint8_t* pa = dm_lds + (buf + saoff + s2 * (TL_ROWS * 4));
    const uint8_t* pb = dm_lds + (buf + sboff + s2 * (TL_ROWS * 4));
#pragma unroll
    for (int i = 0; i < 2; ++i) sa[slot][i] = *(const uint32_t*)(pa + i * 128);
#pragma unroll
    for (int j = 0; j < 4; ++j) sb[slot][j] = *(const uint32_t*)(pb + j * 128);
  };

  f16v acc[2][4];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  // b0, b1, b2: byte offsets of the buffers of stages d, d + 1, d + 2
  uint32_t b0 = 0, b1 = D4_STAGE, b2 = 2 * D4_STAGE;
  request(0, b0);
  request(1, b1);
#pragma unroll
  for (int part = 0; part < 4; ++part) request_part(2, b2, part);
  __builtin_amdgcn_s_waitcnt(waitcnt_vm(D4_LOADS + 4));  // stage 0 has landed
  __syncthreads();
  read_ops(0, b0, 0);
  read_scales(0, b0, 0);
#pragma unroll 1
  for (int d = 0; d < stages; ++d) {
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      // step u = half u / 2, MFMA u % 2 of it; operand slot u % 2, scale slot (u / 2) % 2
      if (u == 3) {
        // every LDS read of stage d has been issued: once all waves are here its buffer
        // can take stage d + 3, and stage d + 1 has landed for everyone
        __builtin_amdgcn_s_waitcnt(waitcnt_vm(D4_LOADS));
        __syncthreads();
#pragma unroll
        for (int part = 0; part < 4; ++part) request_part(d + 3, b0, part);
        __builtin_amdgcn_sched_barrier(0);
        read_ops(0, b1, 0);
        read_scales(0, b1, 0);
      } else {
#pragma unroll
        for (int part = 4 * u + 4; part < 4 * u + 8; ++part)
          if (part < D4_LOADS) request_part(d + 2, b2, part);
        __builtin_amdgcn_sched_barrier(0);
        read_ops((u + 1) & 1, b0, u + 1);
        if (u == 1) read_scales(1, b0, 1);
      }
      const int sh = 16 * (u & 1) + 8 * h, ss = u >> 1;
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          acc[i][j] = mfma_fp4_32(wv[u & 1][i], sa[ss][i] >> sh, xv[u & 1][j], sb[ss][j] >> sh, acc[i][j]);
      __builtin_amdgcn_sched_barrier(0);
    }
    const uint32_t first = b0;
    b0 = b1;
    b1 = b2;
    b2 = first;
  }
  __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));  // nothing may still be writing LDS at exit

  // lane: m = tile row r, n = 8 q + 4 h + e of each 32 x 32 tile; whole tiles leave
  // through LDS as full 128-byte lines
  const bool whole = m0 + TL_TM <= M && n0 + TL_TN <= N && (N & 7) == 0 && ((uintptr_t)c & 15) == 0;
  if (whole) {
    constexpr int PITCH = 144;
    __syncthreads();  // no wave reads a stage buffer any more, no load is landing in one
    uint8_t* mine = dm_lds + wave * (TL_TM * PITCH);
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          h4 out;
#pragma unroll
          for (int e = 0; e < 4; ++e) out[e] = (_Float16)acc[i][j][4 * q + e];
          *(h4*)(mine + (j * 32 + r) * PITCH + i * 64 + q * 16 + h * 8) = out;
        }
    w4_half* cw = c + (size_t)m0 * N + n0 + wave * 64;
#pragma unroll
    for (int it = 0; it < TL_TM / 8; ++it) {
      const int row = it * 8 + (lane >> 3), piece = lane & 7;
      const u4 v = *(const u4*)(mine + row * PITCH + piece * 16);
      *(u4*)(cw + (size_t)row * N + piece * 8) = v;
    }
    return;
  }
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int m = m0 + j * 32 + r;
    if (m >= M) continue;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int nn = n0 + wave * 64 + i * 32 + 8 * q + 4 * h;
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

// Worth it once the tile grid covers a good part of the chip; below that the
// skinny kernel's grid.y walk is faster (measured at K = 4096: N = 4096, M = 256
// -> 32 tiles 37 us here, 23 us there; M = 512 -> 64 tiles 31 us here; N = 14336,
// M = 256 -> 112 tiles 34 us here, 54 us there).  x_row_bytes: K/2 or K.
bool tile_applies(const w4_packed_mx_view& w, const void* xq, const uint8_t* xs, int M,
                  int x_row_bytes) {
  const long long tiles = (long long)((w.N + TL_TN - 1) / TL_TN) * ((M + TL_TM - 1) / TL_TM);
  return M >= 128 && tiles >= 64 && w.K % 256 == 0 && (long long)w.N * w.K < (1LL << 32) &&
         (long long)M * x_row_bytes < (1LL << 32) && ((uintptr_t)w.q & 15) == 0 &&
         ((uintptr_t)xq & 15) == 0 && ((uintptr_t)w.scales & 7) == 0 && ((uintptr_t)xs & 7) == 0;
}

template <bool XF8>
hipError_t launch_tile(const w4_packed_mx_view& w, const void* xq, const uint8_t* xs, int M,
                       w4_half* c, hipStream_t s) {
  const int tiles_n = (w.N + TL_TN - 1) / TL_TN, tiles_m = (M + TL_TM - 1) / TL_TM;
  if ((long long)tiles_n * tiles_m > 0x7FFFFFFFLL) return hipErrorInvalidConfiguration;
  // more than 64 KB of LDS has to be granted per device, once
  static std::atomic<bool> granted[64] = {};
  int dev = 0;
  if (hipError_t e = hipGetDevice(&dev); e != hipSuccess) return e;
  const bool grant = dev < 0 || dev >= 64 || !granted[dev];
  if constexpr (XF8) {
    constexpr int lds_bytes = Dm<true>::STAGES * Dm<true>::STAGE;
    if (grant) {
      const hipError_t e = hipFuncSetAttribute((const void*)mxn_tile_dma_kernel<true>,
                                               hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
      if (e != hipSuccess) return e;
    }
    mxn_tile_dma_kernel<true><<<dim3((unsigned)(tiles_n * tiles_m)), dim3(DM_THREADS), lds_bytes, s>>>(
        w.q, w.scales, (const uint32_t*)xq, xs, c, w.N, w.K, w.B, M, tiles_n, tiles_m);
  } else {
    constexpr int lds_bytes = D4_STAGES * D4_STAGE;
    if (grant) {
      const hipError_t e = hipFuncSetAttribute((const void*)mxn_tile4_kernel,
                                               hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
      if (e != hipSuccess) return e;
    }
    mxn_tile4_kernel<<<dim3((unsigned)(tiles_n * tiles_m)), dim3(D4_THREADS), lds_bytes, s>>>(
        w.q, w.scales, (const uint32_t*)xq, xs, c, w.N, w.K, w.B, M, tiles_n, tiles_m);
  }
  if (dev >= 0 && dev < 64) granted[dev] = true;
  return hipGetLastError();
}

}  // namespace

hipError_t launch_gemm_mx_w4a4(const w4_packed_mx_view& w, const w4_packed_mx_view& x,
                               w4_half* c, hipStream_t s) {
  if (tile_applies(w, x.q, x.scales, x.N, w.K / 2)) return launch_tile<false>(w, x.q, x.scales, x.N, c, s);
  return launch_skinny<false>(w, x.q, x.scales, x.N, c, s);
}

// E4M3 activations (K a multiple of 32, rows 16-byte aligned).
hipError_t launch_gemm_mx_w4a8(const w4_packed_mx_view& w, const w4_act_mx8_view& x, w4_half* c,
                               hipStream_t s) {
  if (tile_applies(w, x.q, x.scales, x.M, w.K)) return launch_tile<true>(w, x.q, x.scales, x.M, c, s);
  return launch_skinny<true>(w, x.q, x.scales, x.M, c, s);
}

}  // namespace w4k
