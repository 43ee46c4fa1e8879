// Decode-batch W4A16 GEMM for M <= 16 with the activations fetched once per
// workgroup: c[M,N] = X[M,K] * dequant(W)[N,K]^T, K = 2048 or 4096 (mma.cuh:63-230 is
// the reference's kernel for this path; it stages x in shared memory per block).
//
// At these shapes a 16-row tile of W is 16 KB to 32 KB of codes, and the MFMAs
// that consume it want 64 KB to 128 KB of FP16 activations as operands.  With one
// tile per workgroup the activations, not the weights, were what the memory path
// spent its time on (measured at M = 8, N = 11008, K = 4096: 15.1 us; with constant
// activations 9.0 us; with constant weights instead 11.3 us).  So a workgroup
// takes T tiles and brings its activations in once:
//   * 8 waves split K (wave w owns k in [K/8 w, K/8 (w + 1))), as in the kernels of
//     gemm_mfma.hip; a wave needs only its own slice of x.
//   * global_load_lds_dwordx4 moves that slice into the wave's own 8 or 16 KB of
//     LDS: a load instruction takes 4 rows x 256 contiguous bytes (whole cache
//     lines; operand loads straight into registers would take 64 bytes of each of
//     16 rows), pieces XOR-swizzled by the row so that the reads back are
//     conflict-free.  No other wave touches the region: no barrier.
//   * the slice is read back once into registers as MFMA B operands and serves
//     all T tiles; the codes of all T tiles are requested before anything is
//     consumed.
//   * a word is expanded in natural k order (see gemm_tile_dma.hip) straight into
//     the A operand of v_mfma_f32_16x16x32_f16.
// Partial sums of the eight waves meet in LDS in wave order (no atomics).
#include <atomic>

#include "dq.cuh"
#include "kernels.h"

namespace w4k {
namespace {

typedef __attribute__((address_space(3))) void* lds_ptr;
constexpr int DR_WAVES = 8, DR_THREADS = 64 * DR_WAVES;
constexpr int waitcnt_vm(int n) { return (n & 0xF) | ((n >> 4) << 14) | 0x0F70; }
extern __shared__ __attribute__((aligned(16))) uint8_t dr_lds[];

// Eight codes of a packed word -> eight FP16 weights in k order.  cneg: packed
// {-(1024 + z), -(64 + z)}; s2: the group scale in both halves; mask, magic:
// 0x00F0000F and 0x54006400 in registers.
__device__ __forceinline__ h8 expand_word(uint32_t w, h2 cneg, h2 s2, uint32_t mask, uint32_t magic) {
  u4 out;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const uint32_t p = __builtin_amdgcn_perm(0u, w, 0x0c000c00u | (uint32_t)(i << 16) | (uint32_t)i);
    const uint32_t v = (p & mask) | magic;
    out[i] = as_u32((as_h2(v) + cneg) * s2);
  }
  return __builtin_bit_cast(h8, out);
}

// FMT: 0 W4 symmetric, 1 W4 with zero-points, 2 MXFP4.  K = 1024 CH.  POW2: gs is a
// power of two (shift gs_shift); GSV: 1, 2, 3 for gs = 128, 64, 32 with scale arrays
// (4: gs a power of two from 128 on at long K, scales loaded one by one: a chunk lies in one group)
// aligned for vector loads, else 0.  T tiles of 16 rows per
// workgroup: tile g + gridDim.x t for t < T (tiles past the end are computed on
// the last tile's rows and not stored).  MT tiles of 16 activation rows (M <= 16 MT).
//
// CPV, if not 0, chunks of x per phase: two at MT = 1 halve the region to 8 KB, so that a
// compute unit holds two workgroups when the grid has more of them than compute units
// (N = 28672, K = 4096, M = 8: 18.7 -> 17.2 us; on one-round grids the same split is slower,
// 8.5 -> 9.5 us at N = 11008).
// A wave's LDS region holds 16 KB: with MT > 1 its slice of x goes through it in MT
// phases of CP = 4 / MT chunks of 128 k (all MT row tiles of a chunk at a time); the
// next phase is requested as soon as the current one sits in registers, so it
// lands while the current one multiplies.
template <int FMT, int CH, bool POW2, int GSV, int T, int MT, int CPV = 0>
__global__ __launch_bounds__(DR_THREADS) void mfma_decode_resident_kernel(
    const WView p, const w4_half* __restrict__ x, w4_half* __restrict__ c, const int M,
    const int gs_shift, const int tiles) {
  constexpr bool MX = FMT == 2;
  // LATE (gs = 128: a wave's 128-k chunk is one group): the scale is applied to the chunk's
  // FP32 sums, not to the weights.  The operands swap roles (A = x, B = W) so that a lane's
  // four sums belong to its own row of W and take that row's scale: sum[e] += s_r * chunk[e].
  // Symmetric weights: the MFMA operand is the biased code itself, (1024 + q) for even k and
  // (64 + q) for odd k -- what one mask-and-or makes of a byte, exact in FP16 -- and the
  // chunk's accumulator starts at -sum_k x_k (b_k + 8), which one more MFMA chain per chunk
  // (x times the constant biases) gives for all tiles at once: 8 vector instructions per
  // word instead of 16.  With zero-points the operand is q - z (one packed add more: 12 per
  // word; the zero-point's share through a chain of its own measured no faster).  Outputs
  // differ from the per-weight arithmetic by FP32 rounding only (the hooked calls keep that).
  // (not with four activation row tiles: their sixteen MFMAs per chunk already keep the
  // matrix pipe as busy as the expansion keeps the vector pipe, the extra chains would
  // make it the longer of the two, and the chunk sums do not fit the register file beside
  // three tiles of codes)
  // (nor where two tiles of fourteen chunks and two row tiles leave no registers for the chunk sums)
  constexpr bool LATE = !MX && (GSV == 1 || GSV == 4) && MT <= 2 && !(CH == 14 && T == 2 && MT == 2);
  // K: any multiple of 128 with ceil(K / 128 / 8) == CH; wave w owns the 128-k chunks
  // [CH w, CH (w + 1)) that exist (the last waves may own fewer: chunks past the end
  // are fetched from a clamped address and meet zero activations)
  const int K = p.K, WPR = K >> 3, nchunks = K >> 7;
  constexpr bool EXACT = CH == 2 || CH == 4;  // K = 1024 CH by the launcher: every chunk exists
  constexpr int CP = CPV ? CPV : (4 / MT) < CH ? (4 / MT) : CH;  // chunks per phase
  constexpr int PH = (CH + CP - 1) / CP;              // phases (the last may be partial)
  constexpr int XBYTES = MT * CP * 4096;              // the wave's LDS region
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r = lane & 15, b = lane >> 4;
  const int kw = wave * (128 * CH) + 32 * b;  // first k of this lane
  // chunk i of this wave, clamped to the last one of the row
  auto chunk_k = [&](int i) {
    const int cidx = wave * CH + i;
    return (EXACT || cidx < nchunks) ? kw + 128 * i : (nchunks - 1) * 128 + 32 * b;
  };
  const int m0 = (int)blockIdx.y * (16 * MT);  // grid.y walks the activation rows 16 MT at a time

  // rows of W this lane reads, per tile
  size_t nrow[T];
#pragma unroll
  for (int t = 0; t < T; ++t) {
    const int tile = min((int)blockIdx.x + (int)gridDim.x * t, tiles - 1);
    nrow[t] = (size_t)(tile * 16 + r);
  }
  // Scales: a lane's CH chunks lie 128 k apart; chunk i of lane group b is group
  // (CH wave + i) (128 / gs) + b / (gs / 32) of the row.  With gs = 128, 64 or 32 (GSV)
  // the wave's groups are CH, 2 CH or 4 CH consecutive FP16 scales: one or two vector
  // loads and a per-lane pick, and their zero-points sit in one or two words;
  // MXFP4's CH bytes are 4 apart in 4 CH consecutive ones.  Other group sizes load
  // them one by one.
  constexpr bool VEC = (MX && EXACT) || (GSV != 0 && GSV != 4);
  constexpr int PER = MX ? 4 : GSV == 1 ? 1 : GSV == 2 ? 2 : 4;  // groups per 128-k chunk
  uint32_t sc[T][CH], zw[T][CH];
  int gidx[CH];
#pragma unroll
  for (int i = 0; i < CH; ++i) {
    const int k = chunk_k(i);
    gidx[i] = MX ? (k >> 5) : GSV == 1 ? wave * CH + i  // (one group per chunk: the same for every lane)
              : (GSV && GSV != 4) ? (k >> (8 - GSV)) : POW2 ? (k >> gs_shift) : k / p.gs;
  }
  // Codes.  The operand layout wants lane (r, b) to hold row r, 32 k of chunk i: fetched
  // as such, a load instruction takes 64 bytes of each of 16 rows, half of every
  // 128-byte line it touches, and the memory path moves those at 0.8 of the rate of
  // whole lines (measured with loads alone on this grid).  So with an even number of
  // chunks (and rows that are whole lines) the two loads of chunks 2P, 2P + 1 take whole
  // lines instead: load 2P rows 0..7 of the tile, load 2P + 1 rows 8..15; lane (r, b)
  // fetches piece b + 4 (r / 8) of its line in the first and piece b + 4 (1 - r / 8) in
  // the second.  A lane then holds its own row's piece of chunk 2P in one register set
  // and, in the other, the piece of chunk 2P + 1 that lane r ^ 8 wants: pair_fix()
  // selects and rotates the rows of 16 lanes by 8, which restores the layout above.
  constexpr bool PAIRC = CH % 2 == 0;
  const bool paired = PAIRC && (EXACT || (K & 255) == 0);
  u4 qw[T][CH];
  auto load_tile = [&](int t) {
    if (paired) {
      const uint32_t* qa = p.q + (nrow[t] - (size_t)(r & 8)) * WPR;  // row r % 8 of the tile
      const uint32_t* qb = qa + (size_t)8 * WPR;                     // row 8 + r % 8
      const int pa = 4 * (b + 4 * (r >> 3)), pb = 4 * (b + 4 * ((r >> 3) ^ 1));  // piece, in words
#pragma unroll
      for (int i = 0; i + 1 < CH; i += 2) {
        const int cidx = wave * CH + i;
        const int w0 = 16 * ((EXACT || cidx < nchunks) ? cidx : nchunks - 2);
        qw[t][i] = __builtin_nontemporal_load((const u4*)(qa + w0 + pa));
        qw[t][i + 1] = __builtin_nontemporal_load((const u4*)(qb + w0 + pb));
      }
    } else {
      const uint32_t* qr = p.q + nrow[t] * WPR;
#pragma unroll
      for (int i = 0; i < CH; ++i)
        qw[t][i] = __builtin_nontemporal_load((const u4*)(qr + (chunk_k(i) >> 3)));
    }
  };
  auto pair_fix = [&](int t, int i) {  // chunks i, i + 1 (i even)
    if (!paired) return;
    const bool lo = r < 8;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const uint32_t a = qw[t][i][e], bb = qw[t][i + 1][e];
      qw[t][i][e] = lo ? a : bb;
      // row_ror:8 -- lane r of each row of 16 takes the value of lane r ^ 8
      qw[t][i + 1][e] = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)(lo ? bb : a), 0x128, 0xF, 0xF, true);
    }
  };
  auto load_scales = [&](int t) {
    if constexpr (MX && !EXACT) {
#pragma unroll
      for (int i = 0; i < CH; ++i) sc[t][i] = ((const uint8_t*)p.scales)[nrow[t] * p.B + gidx[i]];
    } else if constexpr (MX) {  // bytes 4 CH wave .. + 4 CH - 1 of the row; this lane's are b + 4 i
      const uint8_t* sp = (const uint8_t*)p.scales + nrow[t] * p.B + wave * (4 * CH);
      uint32_t w[CH];
      if constexpr (CH == 4) {
        const u4 v = *(const u4*)sp;
#pragma unroll
        for (int i = 0; i < CH; ++i) w[i] = v[i];
      } else {
        const u2 v = *(const u2*)sp;
#pragma unroll
        for (int i = 0; i < CH; ++i) w[i] = v[i];
      }
#pragma unroll
      for (int i = 0; i < CH; ++i) sc[t][i] = (w[i] >> (8 * b)) & 0xFFu;
    } else if constexpr (VEC) {
      // HALVES consecutive scales = HALVES / 2 dwords; this lane's scale of chunk i is
      // half PER i + (b >> (GSV == 2 ? 1 : 0 ...)) of them
      constexpr int HALVES = PER * CH, DW = HALVES / 2;
      const uint32_t* sp = (const uint32_t*)((const uint16_t*)p.scales + nrow[t] * p.G + wave * HALVES);
      uint32_t w[DW];
      if constexpr (DW == 1) {
        w[0] = *sp;
      } else if constexpr (DW == 2) {
        const u2 v = *(const u2*)sp;
        w[0] = v[0], w[1] = v[1];
      } else if constexpr (DW == 8) {
        // 32 bytes per row: the lower 32 lanes fetch the first 16, the upper 32 the
        // second 16, and v_permlane32_swap hands each half the other's -- one load
        // instruction that touches 16 lines instead of two that touch 16 each
        const u4 v = *(const u4*)(sp + 4 * (lane >> 5));
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const auto pr = __builtin_amdgcn_permlane32_swap(v[e], v[e], false, false);
          w[e] = pr[0];      // lanes 0..31: own, lanes 32..63: that of lane - 32
          w[4 + e] = pr[1];  // lanes 0..31: that of lane + 32, lanes 32..63: own
        }
      } else {
#pragma unroll
        for (int q = 0; q < DW / 4; ++q) {
          const u4 v = *(const u4*)(sp + 4 * q);
#pragma unroll
          for (int e = 0; e < 4; ++e) w[4 * q + e] = v[e];
        }
      }
      const int sub = GSV == 1 ? 0 : GSV == 2 ? (b >> 1) : b;  // group of the chunk this lane is in
#pragma unroll
      for (int i = 0; i < CH; ++i) {
        // half index PER i + sub: dword (PER i + sub) / 2, upper half if odd
        uint32_t d;
        // (a bitwise select: written as a conditional the compiler indexed the array
        // with the condition, which put it in scratch memory -- two stores and four
        // dependent loads per tile through the memory path, 1.8 us per call at gs = 32)
        if constexpr (PER == 4) d = w[2 * i] ^ ((w[2 * i] ^ w[2 * i + 1]) & (0u - (uint32_t)((sub >> 1) & 1)));
        else if constexpr (PER == 2) d = w[i];
        else d = w[i >> 1];
        const bool hi = PER == 1 ? (i & 1) : (sub & 1);
        sc[t][i] = hi ? (d >> 16) : (d & 0xFFFFu);
      }
      if (FMT == 1) {
        // groups PER CH wave .. + PER CH - 1: one zero-point word per eight
        constexpr int ZW = (HALVES + 7) / 8;
        const uint32_t* zp = p.zeros + nrow[t] * words(p.G) + ((wave * HALVES) >> 3);
        uint32_t z[ZW];
        if constexpr (ZW == 2) {
          const u2 v = *(const u2*)zp;
          z[0] = v[0], z[1] = v[1];
        } else {
          z[0] = *zp;
        }
#pragma unroll
        for (int i = 0; i < CH; ++i) zw[t][i] = z[ZW == 2 ? (i >> 1) : 0];
      }
    } else {
#pragma unroll
      for (int i = 0; i < CH; ++i) {
        sc[t][i] = ((const uint16_t*)p.scales)[nrow[t] * p.G + gidx[i]];
        if (FMT == 1) zw[t][i] = p.zeros[nrow[t] * words(p.G) + (gidx[i] >> 3)];
      }
    }
  };
  static_assert(EXACT || GSV == 0 || GSV == 4, "vector scale loads assume K = 1024 CH");
  static_assert(GSV != 4 || POW2, "chunk-wise scaling at long K: gs a power of two from 128 on");

  // Phase ph of this wave's slice of x -> its LDS region: block (mt, cc, rq) = rows
  // 16 mt + 4 rq .. + 3 of the 128-k chunk CP ph + cc; lane l fetches row l/16 of the
  // four, 16-byte piece (l%16) ^ (row % 16) of the chunk's 256 bytes.  Rows past M
  // repeat row M - 1 (their columns of the product are never stored).
  const uint32_t region = (uint32_t)(uintptr_t)(lds_ptr)dr_lds + (uint32_t)wave * XBYTES;
  const char* xb = (const char*)x;
  auto request_x = [&](int ph) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int cc = 0; cc < CP; ++cc)
#pragma unroll
        for (int rq = 0; rq < 4; ++rq) {
          if (ph * CP + cc >= CH) continue;
          // quads of activation rows that do not exist are not fetched (with one row tile:
          // M = 8 moves half, M = 4 a quarter of a tile's 128 KB through L2 -> LDS); their
          // columns of the product are never stored, whatever the region holds there
          if (MT == 1 && m0 + 4 * rq >= M) continue;
          const int r16 = 4 * rq + (lane >> 4), row = m0 + 16 * mt + r16;
          const int cidx = wave * CH + ph * CP + cc;  // a chunk past the end repeats the last one
          const uint32_t off = (uint32_t)min(row, M - 1) * (uint32_t)(K * 2) +
                               (uint32_t)((EXACT || cidx < nchunks) ? cidx : nchunks - 1) * 256u +
                               (uint32_t)(((lane & 15) ^ r16) * 16);
          const uint32_t dst = region + (uint32_t)((mt * CP + cc) * 4 + rq) * 1024u;
          asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1"
                       :
                       : "v"(off), "s"(xb), "s"(dst)
                       : "memory", "m0");
        }
  };
  // Requests, in the order the memory path will serve them.  The codes of tile t + 1
  // are requested just before tile t is multiplied, not all up front: a compute
  // unit's eight waves ask for more than its memory path holds, a wave stands still
  // at a load until the path takes it, and a wave that had to place every tile's
  // loads first would start its arithmetic only when most of the stream has gone by
  // (measured: half of the waves after 3.5 of 7.3 us, the last one with all T tiles
  // still to expand).  With several tiles the activations go first and a barrier
  // keeps any wave's codes from overtaking another wave's activations, so that every
  // wave can start on tile 0 early; with one tile there is nothing to overlap and the
  // codes, which come from HBM, go first.
  if (T == 1) load_tile(0);
  request_x(0);
  if (T > 1) {
    // (with at most eight activation rows the two or fewer quads a wave fetches are too
    // little to be worth holding the codes back for: N = 11008, M = 8: 8.15 -> 8.0 us without
    // the barrier; with sixteen rows it is worth 0.1 us)
    if (MT > 1 || m0 + 8 < M) {
      __builtin_amdgcn_sched_barrier(0);
      __builtin_amdgcn_s_barrier();
      __builtin_amdgcn_sched_barrier(0);
    }
    load_tile(0);
  }
#pragma unroll
  for (int t = 0; t < T; ++t) load_scales(t);
  if (T > 1) load_tile(1);
  __builtin_amdgcn_sched_barrier(0);  // every request above is issued before the wait below

  uint32_t mask = 0x00F0000Fu, magic = 0x54006400u;
  asm volatile("" : "+s"(mask));   // opaque: as literals they cost two instructions
  asm volatile("" : "+v"(magic));  // instead of one and-or
  f4 acc[T][MT];
#pragma unroll
  for (int t = 0; t < T; ++t)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[t][mt] = f4{0.f, 0.f, 0.f, 0.f};

#pragma unroll
  for (int ph = 0; ph < PH; ++ph) {
    // Phase 0 has landed once at most the loads issued after it are outstanding;
    // later phases are the youngest requests of the wave.
    if (ph == 0) __builtin_amdgcn_s_waitcnt(waitcnt_vm(T > 1 ? CH : 0));
    else __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
    // B operands: MFMA j of chunk i contracts k = kw + 128 i + 8 j .. + 7 = piece 4 b + j
    u4 xv[MT][CP][4];
    {
      const uint8_t* mine = dr_lds + wave * XBYTES;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int cc = 0; cc < CP; ++cc)
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            if (ph * CP + cc >= CH) continue;
            xv[mt][cc][j] = *(const u4*)(mine + ((mt * CP + cc) * 4 + (r >> 2)) * 1024 +
                                         ((r & 3) * 16 + ((4 * b + j) ^ r)) * 16);
            if (!EXACT && wave * CH + ph * CP + cc >= nchunks) xv[mt][cc][j] = u4{0u, 0u, 0u, 0u};
          }
    }
    if (ph + 1 < PH) {
      // the region is free once these reads have returned: ask for the next phase now
      __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
      __builtin_amdgcn_sched_barrier(0);
      request_x(ph + 1);
    }
    // LATE, symmetric: what every chunk's sums start from, for all tiles: -sum_k x_k (b_k + 8),
    // the same in every column
    [[maybe_unused]] f4 negb[MT][CP];
    if constexpr (LATE && FMT == 0) {
      const uint32_t nb = 0xD480E408u;  // -(1024 + 8) | -(64 + 8)
      const h8 nbv = __builtin_bit_cast(h8, u4{nb, nb, nb, nb});
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int cc = 0; cc < CP; ++cc) {
          negb[mt][cc] = f4{0.f, 0.f, 0.f, 0.f};
          if (ph * CP + cc >= CH) continue;
#pragma unroll
          for (int j = 0; j < 4; ++j)
            negb[mt][cc] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, xv[mt][cc][j]), nbv,
                                                                  negb[mt][cc], 0, 0, 0);
        }
    }
#pragma unroll
    for (int t = 0; t < T; ++t) {
      if (ph == 0 && t >= 1) {
        // request tile t + 1, then wait for tile t: what was requested after it may
        // still be out (after tile 1: the second phase of x, and tile 2)
        constexpr int NX1 = PH > 1 ? MT * (CP < CH - CP ? CP : CH - CP) * 4 : 0;
        static_assert(NX1 + CH < 64, "vmcnt is a 6-bit counter");
        __builtin_amdgcn_sched_barrier(0);
        if (t + 1 < T) load_tile(t + 1);
        __builtin_amdgcn_sched_barrier(0);
        // (only the tile's first pair of chunks has to be here: the rest of it lands while
        // that pair is expanded -- the compiler places the waits for the later registers --
        // so the last tile's arithmetic, which nothing overlaps, starts half a tile earlier)
        constexpr int LATER = (PAIRC && CH >= 4) ? CH - 2 : 0;
        static_assert(NX1 + CH + LATER < 64, "vmcnt is a 6-bit counter");
        if (t == 1) __builtin_amdgcn_s_waitcnt(waitcnt_vm(NX1 + (T > 2 ? CH : 0) + LATER));
        else if (t + 1 < T) __builtin_amdgcn_s_waitcnt(waitcnt_vm(CH + LATER));
        else __builtin_amdgcn_s_waitcnt(waitcnt_vm(LATER));
      }
#pragma unroll
      for (int cc = 0; cc < CP; ++cc) {
        const int i = ph * CP + cc;
        if (i >= CH) continue;
        if (PAIRC && (i & 1) == 0 && i + 1 < CH) pair_fix(t, i);
        if constexpr (LATE) {
          const float s32 = half_bits_to_float(sc[t][i]);
          f4 part[MT];
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) part[mt] = FMT == 1 ? f4{0.f, 0.f, 0.f, 0.f} : negb[mt][cc];
          [[maybe_unused]] h2 cneg;
          if (FMT == 1) {
            const uint32_t z = (zw[t][i] >> (4 * (gidx[i] & 7))) & 0xFu;
            cneg = as_h2(0xD400E400u | (z << 20) | z);
          }
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            u4 a;
#pragma unroll
            for (int e = 0; e < 4; ++e)
              a[e] = (__builtin_amdgcn_perm(0u, qw[t][i][j], 0x0c000c00u | (uint32_t)(e << 16) | (uint32_t)e) & mask) | magic;
            if (FMT == 1) {
#pragma unroll
              for (int e = 0; e < 4; ++e) a[e] = as_u32(as_h2(a[e]) + cneg);
            }
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
              part[mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, xv[mt][cc][j]),
                                                                __builtin_bit_cast(h8, a), part[mt], 0, 0, 0);
          }
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) {
            acc[t][mt] += part[mt] * s32;
          }
        } else {
        h2 cneg, s2;
        float sf = 0.f;
        if (MX) {
          sf = mx_scale(sc[t][i]);
        } else {
          const uint32_t z = FMT == 1 ? ((zw[t][i] >> (4 * (gidx[i] & 7))) & 0xFu) : 8u;
          cneg = as_h2(0xD400E400u | (z << 20) | z);
          s2 = splat_bits(sc[t][i]);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          h8 a;
          if (MX) {
            h2 n4[4];
            dq_mx(qw[t][i][j], sf, n4);
            a = __builtin_bit_cast(h8, u4{as_u32(n4[0]), as_u32(n4[1]), as_u32(n4[2]), as_u32(n4[3])});
          } else {
            a = expand_word(qw[t][i][j], cneg, s2, mask, magic);
          }
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
            acc[t][mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, __builtin_bit_cast(h8, xv[mt][cc][j]),
                                                                acc[t][mt], 0, 0, 0);
        }
        }
      }
    }
  }

  // Fixed-order combine of the 8 K slices.  The x regions are free once every wave
  // is here; entry (t, mt) of wave w goes to red[w][t MT + mt]; wave w then sums
  // the entries e = w, w + 8, ... in wave order and stores them.
  constexpr int E = T * MT;
  static_assert(E * 1024 <= XBYTES || E <= 8 * (XBYTES / 1024) , "reduction buffer fits the x regions");
  __syncthreads();
  f4* red = (f4*)dr_lds;  // [DR_WAVES][E][64]
#pragma unroll
  for (int t = 0; t < T; ++t)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) red[(wave * E + t * MT + mt) * 64 + lane] = acc[t][mt];
  __syncthreads();
  for (int e = wave; e < E; e += DR_WAVES) {
    const int t = e / MT, mt = e % MT;
    const int tile = (int)blockIdx.x + (int)gridDim.x * t;
    if (tile >= tiles) continue;
    f4 s = red[e * 64 + lane];
#pragma unroll
    for (int w = 1; w < DR_WAVES; ++w) s += red[(w * E + e) * 64 + lane];
    if constexpr (LATE) {  // lane: weight row 16 tile + r, activation rows 4 b .. + 3 of the row tile
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const int m = m0 + 16 * mt + 4 * b + k;
        if (m < M) c[(size_t)m * p.N + tile * 16 + r] = __builtin_bit_cast(uint16_t, (_Float16)s[k]);
      }
      continue;
    }
    const int m = m0 + 16 * mt + r;
    if (m < M) {  // lane: activation row m, weight rows 16 tile + 4 b .. + 3
      uint16_t hv[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const _Float16 hh = (_Float16)s[k];
        hv[k] = __builtin_bit_cast(uint16_t, hh);
      }
      *(u2*)(c + (size_t)m * p.N + tile * 16 + 4 * b) =
          u2{hv[0] | ((uint32_t)hv[1] << 16), hv[2] | ((uint32_t)hv[3] << 16)};
    }
  }
}

// How the scales are fetched: 1, 2, 3 for gs = 128, 64, 32 at K = 2048 / 4096 with arrays
// aligned for the vector loads of the scales (and of two zero-point words), else 0.
int resident_gsv(const WView& v) {
  // long K (any other K this kernel takes): 4 where a chunk lies in one group, scales loaded one by one
  if (v.K != 2048 && v.K != 4096) return (!v.mx && v.gs >= 128 && (v.gs & (v.gs - 1)) == 0) ? 4 : 0;
  if (!v.mx && (v.K == 2048 || v.K == 4096) && ((uintptr_t)v.scales & 15) == 0 &&
      (v.symmetric || ((uintptr_t)v.zeros & 7) == 0))
    return v.gs == 128 ? 1 : v.gs == 64 ? 2 : v.gs == 32 ? 3 : 0;
  return 0;
}

// Chunks of 128 k per wave for the K this kernel is built for, else 0: K = 2048 and
// 4096 exactly, and any multiple of 128 whose eighth rounds up to 8, 11 or 14 chunks
// (7296 .. 8192, 10368 .. 11264, 13440 .. 14336: the long sides of the usual MLP shapes).
int resident_chunks(int K) {
  if (K == 2048) return 2;
  if (K == 4096) return 4;
  if (K % 128) return 0;
  const int per_wave = (K / 128 + DR_WAVES - 1) / DR_WAVES;
  return (per_wave == 8 || per_wave == 11 || per_wave == 14) ? per_wave : 0;
}

int device_cus();

template <int FMT, int CH, bool POW2, int GSV, int T, int MT, int CPV>
hipError_t launch_t_impl(const WView& v, const w4_half* x, w4_half* c, int M, hipStream_t s, int sh,
                         int tiles, unsigned grid) {
  constexpr int CP = CPV ? CPV : (4 / MT) < CH ? (4 / MT) : CH;
  constexpr int lds_bytes = DR_WAVES * MT * CP * 4096;
  static_assert(DR_WAVES * T * MT * 1024 <= lds_bytes, "the reduction reuses the x regions");
  // more than 64 KB of LDS has to be granted per device, once
  static std::atomic<bool> granted[64] = {};
  int dev = 0;
  if (hipError_t e = hipGetDevice(&dev); e != hipSuccess) return e;
  if (dev < 0 || dev >= 64 || !granted[dev]) {
    const hipError_t e =
        hipFuncSetAttribute((const void*)mfma_decode_resident_kernel<FMT, CH, POW2, GSV, T, MT, CPV>,
                            hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
    if (e != hipSuccess) return e;
    if (dev >= 0 && dev < 64) granted[dev] = true;
  }
  mfma_decode_resident_kernel<FMT, CH, POW2, GSV, T, MT, CPV>
      <<<dim3(grid, (unsigned)((M + 16 * MT - 1) / (16 * MT))), DR_THREADS, lds_bytes, s>>>(v, x, c, M, sh,
                                                                                          tiles);
  return hipGetLastError();
}

// Most tiles per workgroup that an instantiation holds in registers without spilling
// (from the compiler's register counts): with zero-points, four activation row tiles
// take three tiles; two row tiles with per-chunk scale loads (GSV == 0) take seven.
constexpr int dr_tile_cap(int fmt, int gsv, int mt, int ch = 4) {
  // long K (8, 11 or 14 chunks per wave): two tiles where their codes still fit
  if (ch == 8) return 2;
  if (ch == 11) return (fmt != 0 && mt == 4) ? 1 : 2;
  if (ch == 14) return (fmt != 1 && mt <= 2) ? 2 : 1;
  if (fmt == 1 && mt == 4) return 3;
  if (fmt == 1 && mt == 2 && gsv == 0) return 7;
  if (fmt == 1 && mt == 2 && gsv == 1) return 6;  // the chunk sums' starting values take registers too
  return 8;
}

template <int FMT, int CH, bool POW2, int GSV, int T, int MT, int CPV = 0>
hipError_t launch_t(const WView& v, const w4_half* x, w4_half* c, int M, hipStream_t s, int sh,
                    int tiles, unsigned grid) {
  if constexpr (T > dr_tile_cap(FMT, GSV, MT, CH)) {
    return hipErrorInvalidValue;  // decode_resident_tiles() never asks for it
  } else {
    return launch_t_impl<FMT, CH, POW2, GSV, T, MT, CPV>(v, x, c, M, s, sh, tiles, grid);
  }
}

template <int FMT, int CH, bool POW2, int GSV, int T>
hipError_t launch_mt(const WView& v, const w4_half* x, w4_half* c, int M, hipStream_t s, int sh,
                     int tiles, unsigned grid) {
  if constexpr (CH > 4 && T == 1) {
    // long K, one tile per workgroup: up to 64 rows belong to the pipelined long-K kernel, so
    // only the four-row-tile form exists here (it is correct for fewer rows as well)
    return launch_t<FMT, CH, POW2, GSV, T, 4>(v, x, c, M, s, sh, tiles, grid);
  } else {
    if (M <= 16) {
      if constexpr (CH == 4 && T == 4) {
        // more workgroups than compute units: half the LDS each, two per compute unit
        if ((int)grid > device_cus()) return launch_t<FMT, CH, POW2, GSV, T, 1, 2>(v, x, c, M, s, sh, tiles, grid);
      }
      return launch_t<FMT, CH, POW2, GSV, T, 1>(v, x, c, M, s, sh, tiles, grid);
    }
    if (M <= 32) return launch_t<FMT, CH, POW2, GSV, T, 2>(v, x, c, M, s, sh, tiles, grid);
    return launch_t<FMT, CH, POW2, GSV, T, 4>(v, x, c, M, s, sh, tiles, grid);
  }
}

template <int FMT, int CH, bool POW2, int GSV>
hipError_t launch_ch(const WView& v, const w4_half* x, w4_half* c, int M, hipStream_t s, int sh,
                     int tiles, int T) {
  const unsigned grid = (unsigned)((tiles + T - 1) / T);
  if constexpr (CH > 4) {  // long K: one tile per workgroup, or two that share the activations
    if (T == 2) return launch_mt<FMT, CH, POW2, GSV, 2>(v, x, c, M, s, sh, tiles, grid);
    return launch_mt<FMT, CH, POW2, GSV, 1>(v, x, c, M, s, sh, tiles, grid);
  } else {
    switch (T) {
      case 1: return launch_mt<FMT, CH, POW2, GSV, 1>(v, x, c, M, s, sh, tiles, grid);
      case 2: return launch_mt<FMT, CH, POW2, GSV, 2>(v, x, c, M, s, sh, tiles, grid);
      case 3: return launch_mt<FMT, CH, POW2, GSV, 3>(v, x, c, M, s, sh, tiles, grid);
      case 4: return launch_mt<FMT, CH, POW2, GSV, 4>(v, x, c, M, s, sh, tiles, grid);
      default:
        // five to eight tiles: K = 4096, one activation row tile (decode_resident_tiles())
        if constexpr (CH == 4) {
          if (M <= 16) {
            if (T == 5) return launch_t<FMT, CH, POW2, GSV, 5, 1>(v, x, c, M, s, sh, tiles, grid);
            if (T == 6) return launch_t<FMT, CH, POW2, GSV, 6, 1>(v, x, c, M, s, sh, tiles, grid);
            if (T == 7) return launch_t<FMT, CH, POW2, GSV, 7, 1>(v, x, c, M, s, sh, tiles, grid);
            if (T == 8) return launch_t<FMT, CH, POW2, GSV, 8, 1>(v, x, c, M, s, sh, tiles, grid);
          } else {
            if (T == 5) return launch_t<FMT, CH, POW2, GSV, 5, 2>(v, x, c, M, s, sh, tiles, grid);
            if (T == 6) return launch_t<FMT, CH, POW2, GSV, 6, 2>(v, x, c, M, s, sh, tiles, grid);
            if (T == 7) return launch_t<FMT, CH, POW2, GSV, 7, 2>(v, x, c, M, s, sh, tiles, grid);
            if (T == 8) return launch_t<FMT, CH, POW2, GSV, 8, 2>(v, x, c, M, s, sh, tiles, grid);
          }
        }
        return hipErrorInvalidValue;
    }
  }
}

template <int FMT>
hipError_t launch_fmt(const WView& v, const w4_half* x, w4_half* c, int M, hipStream_t s,
                      int tiles, int T) {
  const bool pow2 = !v.mx && (v.gs & (v.gs - 1)) == 0;
  const int sh = pow2 ? __builtin_ctz((unsigned)v.gs) : 0;
  const int gsv = resident_gsv(v);
#define W4_GO(CHV)                                                                          \
  switch (gsv) {                                                                            \
    case 1: return launch_ch<FMT, CHV, true, 1>(v, x, c, M, s, sh, tiles, T);               \
    case 2: return launch_ch<FMT, CHV, true, 2>(v, x, c, M, s, sh, tiles, T);               \
    case 3: return launch_ch<FMT, CHV, true, 3>(v, x, c, M, s, sh, tiles, T);               \
    default:                                                                                \
      return pow2 ? launch_ch<FMT, CHV, true, 0>(v, x, c, M, s, sh, tiles, T)               \
                  : launch_ch<FMT, CHV, false, 0>(v, x, c, M, s, sh, tiles, T);             \
  }
#define W4_LONG(CHV)                                                                        \
  if (gsv == 4) return launch_ch<FMT, CHV, true, 4>(v, x, c, M, s, sh, tiles, T);           \
  return pow2 ? launch_ch<FMT, CHV, true, 0>(v, x, c, M, s, sh, tiles, T)                   \
              : launch_ch<FMT, CHV, false, 0>(v, x, c, M, s, sh, tiles, T);
  if constexpr (FMT == 2) {  // MXFP4 has one form per K: no group size, no scale-load variants
    switch (resident_chunks(v.K)) {
      case 2: return launch_ch<FMT, 2, false, 0>(v, x, c, M, s, sh, tiles, T);
      case 4: return launch_ch<FMT, 4, false, 0>(v, x, c, M, s, sh, tiles, T);
      case 8: return launch_ch<FMT, 8, false, 0>(v, x, c, M, s, sh, tiles, T);
      case 11: return launch_ch<FMT, 11, false, 0>(v, x, c, M, s, sh, tiles, T);
      case 14: return launch_ch<FMT, 14, false, 0>(v, x, c, M, s, sh, tiles, T);
      default: return hipErrorInvalidValue;
    }
  } else {
    switch (resident_chunks(v.K)) {
      case 2: W4_GO(2)
      case 4: W4_GO(4)
      case 8: W4_LONG(8)
      case 11: W4_LONG(11)
      case 14: W4_LONG(14)
      default: return hipErrorInvalidValue;
    }
  }
#undef W4_LONG
#undef W4_GO
}

// Compute units of the current device (per-device cache); 0 on error.
int device_cus() {
  static std::atomic<int> cached[64] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 0;
  if (dev >= 0 && dev < 64 && cached[dev]) return cached[dev];
  int n = 0;
  if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
  if (dev >= 0 && dev < 64) cached[dev] = n;
  return n;
}

// A K this kernel is built for, whole 16-row tiles, a lane's 32-k slice inside one
// group, 16-byte aligned operands, and M <= 64 -- or up to 256 rows in passes of 64
// (grid.y) as long as the passes together stay under what the large-M kernel
// takes, whose workgroups walk all of K alone.  Returns the tiles per workgroup, 0
// if the shape is not this kernel's.
int decode_resident_tiles(const WView& v, const w4_half* x, const w4_half* c, int M) {
  if (M > 256 || M < 1 || v.N % 16 || resident_chunks(v.K) == 0) return 0;
  if (!v.mx && v.gs % 32) return 0;
  if ((((uintptr_t)v.q | (uintptr_t)x) & 15) || ((uintptr_t)c & 7)) return 0;
  if (v.mx && ((uintptr_t)v.scales & 15)) return 0;  // a slice's scale bytes are one vector load
  if (M > 64) {
    // measured at K = 4096: a pass here 8.6 / 13.7 / 16.5 us at N = 4096 / 11008 / 14336, the
    // large-M kernel on its thinnest grids 25 / 37 / 41 us; both grow with K alike, the
    // fixed part of a pass weighs more at K = 2048
    const double passes = (M + 63) / 64, pass_us = 5.0 + v.N / 1235.0;
    double tile_us = 18.0 + v.N / 590.0;
    // up to 128 rows the large-M kernel has 64 x 128 tiles, which fill the chip from
    // N = 8192 on: 20 - 23 us (MXFP4) and 24 - 25 us (W4) for 65 <= M <= 128 at N = 11008
    // and 14336, where two passes here take 26 and 30 us
    const bool tile_gs = v.mx || v.gs == 32 || v.gs == 64 || v.gs % 128 == 0;  // what that kernel takes
    if (M <= 128 && v.N >= 4096 && v.K == 4096 && tile_gs) tile_us = v.mx ? 21.0 : 24.5;
    if (passes * pass_us >= tile_us * (v.K == 2048 ? 0.8 : 1.0)) return 0;
  }
  const int cus = device_cus();
  if (cus < 1) return 0;
  // tiles per workgroup: enough that one workgroup per compute unit covers N, at
  // most four (more workgroups than compute units beyond that)
  int T = (v.N / 16 + cus - 1) / cus;
  // (five to eight at K = 4096 with one activation row tile, where one round of longer
  // workgroups beats two rounds of four-tile ones: N = 22016 / 28672, the fused gate and up
  // projections of the 11008- and 14336-wide MLPs)
  if (T > 4 && !(T <= 8 && M <= 32 && v.K == 4096)) T = 4;
  // long K: one tile per workgroup, unless there are more tiles than compute units and
  // more than a dozen activation rows: then two tiles share a workgroup's activations,
  // which every workgroup pulls out of L2 in full (K = 8192, M = 64: N = 8192 31.7 -> 24.5 us,
  // N = 28672 105 -> 88; K = 13824, N = 5120 50 -> 35; at N = 4096, one tile per compute unit,
  // halving the workgroups is slower, 23 -> 30 us at K = 11008)
  // (from 13 rows on with symmetric weights: N = K = 8192, M = 16 17.2 -> 15.7 us, M = 12 even, M = 8
  // 13.4 -> 14.8; with zero-points M = 16 is even)
  if (resident_chunks(v.K) > 4) T = (M > (!v.mx && v.symmetric ? 12 : 16) && v.N / 16 > cus) ? 2 : 1;
  // what does not fit the register file (dr_tile_cap)
  const int fmt = v.mx ? 2 : v.symmetric ? 0 : 1, mt = M <= 16 ? 1 : M <= 32 ? 2 : 4;
  const int cap = dr_tile_cap(fmt, resident_gsv(v), M > 64 ? 4 : mt, resident_chunks(v.K));
  if (T > cap) T = cap;
  return T;
}

}  // namespace

bool decode_resident_applies(const WView& v, const w4_half* x, const w4_half* c, int M) {
  return decode_resident_tiles(v, x, c, M) != 0;
}

bool decode_resident_shares_long_k(const WView& v, const w4_half* x, const w4_half* c, int M) {
  return resident_chunks(v.K) > 4 && decode_resident_tiles(v, x, c, M) > 1;
}

// Precondition: decode_resident_applies(v, x, c, M); no hook.
hipError_t launch_decode_resident(const WView& v, const w4_half* x, w4_half* c, int M,
                                  hipStream_t s) {
  const int T = decode_resident_tiles(v, x, c, M);
  if (T == 0) return hipErrorInvalidValue;
  const int tiles = v.N / 16;
  if (v.mx) return launch_fmt<2>(v, x, c, M, s, tiles, T);
  return v.symmetric ? launch_fmt<0>(v, x, c, M, s, tiles, T) : launch_fmt<1>(v, x, c, M, s, tiles, T);
}

}  // namespace w4k
