// The large-M W4A16 GEMM on 256 x 256 workgroup tiles (mma.cuh:234-260 is the reference's
// tensor-core dispatch for these shapes): c[M,N] = X[M,K] * dequant(W)[N,K]^T.
//
// Same scheme as the 128 x 256 kernel of gemm_tile_dma.hip -- packed words and
// activations go global -> LDS with global_load_lds_dwordx4, every wave expands the
// words of its own MFMA operands in registers, v_mfma_f32_32x32x16_f16 accumulates in
// FP32 -- with a wave that holds 64 rows of W against all 256 rows of X: sixteen
// MFMAs share the two words expanded per 16-k step (eight in the smaller kernel), so
// the vector instructions and the LDS bytes per MFMA are half of that kernel's, and a
// grid of M / 256 x N / 256 tiles covers in one round what takes the smaller tiles two.
//   * a wave's 2 x 8 accumulator tiles are 256 registers (the AGPR half of the file:
//     one wave per SIMD has 512);
//   * a stage is 64 k: 32 bytes of a W row, 128 bytes of an X row (one line), 42 KB;
//     three stage buffers, one barrier per stage (64 MFMAs per wave);
//   * the instruction order of the main loop is fixed by hand, MFMA by MFMA: with one wave
//     per SIMD every vector, LDS and load instruction is issued between two MFMAs of the
//     same wave, and a dependent pair back to back costs the wave the first one's latency;
//   * lane l of an MFMA brings row l % 32 and k 32 (l / 32) + 8 u .. + 7 in step u of a
//     stage: its four W words are one 16-byte LDS read per stage and 32-row tile, its X
//     operand is 16-byte piece 4 (l / 32) + u of the row.
// The k order of the additions is that of the 128 x 256 kernel.  No dequant hook here:
// hooked calls stay on that kernel.
#include <atomic>

#include "dq.cuh"
#include "kernels.h"

namespace w4k {
namespace {

typedef float f16v __attribute__((ext_vector_type(16)));
typedef __attribute__((address_space(3))) void* lds_ptr;

constexpr int T2_THREADS = 256, T2_STAGES = 3;
constexpr int T2_W_BYTES = 256 * 32, T2_X_BYTES = 256 * 128;
constexpr int T2_TILE = T2_W_BYTES + T2_X_BYTES;
constexpr int T2_STAGE = T2_TILE + 2 * 256 * 4;  // + a scale dword and a zero-point word per W row
constexpr int T2_C_PITCH = 128 + 16;             // a wave's 64 outputs of one X row, padded
constexpr int T2_C_BYTES = 4 * 256 * T2_C_PITCH;
constexpr int T2_LDS = T2_STAGES * T2_STAGE > T2_C_BYTES ? T2_STAGES * T2_STAGE : T2_C_BYTES;
static_assert(T2_LDS <= 160 * 1024, "stage buffers and the output staging fit LDS");

// s_waitcnt vmcnt(N) alone (gfx9 encoding: vmcnt in [3:0] and [15:14])
constexpr int t2_waitcnt_vm(int n) { return (n & 0xF) | ((n >> 4) << 14) | 0x0F70; }

extern __shared__ __attribute__((aligned(16))) uint8_t t2_lds[];

// Position of 16-byte piece p of X row R in a stage buffer.  A load instruction writes
// lane l's 16 bytes at 16 l, so it covers eight whole rows; which piece a lane fetches
// is chosen so that the sixteen consecutive rows one phase of a ds_read_b128 touches
// (same p) fall on sixteen distinct 16-byte bank groups.
__device__ __forceinline__ int t2_x_key(int R) { return (R >> 1) & 7; }
__device__ __forceinline__ int t2_x_at(int R, int p) {
  return (R >> 3) * 1024 + ((R & 7) * 8 + (p ^ t2_x_key(R))) * 16;
}
// W rows are two pieces each: the 32 rows x 2 pieces a wave reads are one contiguous KB
__device__ __forceinline__ int t2_w_at(int R, int p) { return (R * 2 + p) * 16; }

// FMT: 0 W4 symmetric, 1 W4 with zero-points, 2 MXFP4.  GS32: W4 groups of 32 (a lane's
// 32 k of a stage are one group, the stage two); otherwise gs is a multiple of 64 and
// the stage lies in one group.  G: scales per row (MXFP4: E8M0 bytes per row).
template <int FMT, bool GS32>
__global__ __launch_bounds__(T2_THREADS) void w4_tile256_kernel(
    const uint32_t* __restrict__ wq, const void* __restrict__ scales,
    const uint32_t* __restrict__ zeros, const w4_half* __restrict__ x, w4_half* __restrict__ c,
    int N, int K, int G, int gs, int M, int tiles_n, int tiles_m) {
  constexpr bool ASYM = FMT == 1, MX = FMT == 2;
  constexpr int WAVES = 4;
  constexpr int NI = 2, MJ = 8;                   // 32-row tiles of W and of X per wave
  constexpr int WI = 8 / WAVES, XI = 32 / WAVES;  // 1 KB load instructions of W and of X per wave and stage
  constexpr int LOADS = WI + XI + 1 + (ASYM ? 1 : 0);
  constexpr int CH = NI * MJ / 4;  // chunks of four MFMAs per 16-k step
  static_assert(LOADS <= 4 * CH, "at most one load instruction per chunk");
  const int t = threadIdx.x, lane = t & 63;
  const int wave = __builtin_amdgcn_readfirstlane(t >> 6);  // in an SGPR: LDS addresses go to M0
  const int r = lane & 31, h = lane >> 5;
  // Consecutive workgroup ids land on different XCDs (each with its own L2): give each
  // XCD a block of the tile grid, or failing that a contiguous run of the tile order, m fastest.
  int L = blockIdx.x;
  const int total = tiles_n * tiles_m;
  int tn_i, tm_i;
  if (tiles_n % 4 == 0 && tiles_m % 2 == 0) {
    // XCD x takes a block of tiles_n / 4 x tiles_m / 2 tiles: what its workgroups fetch per
    // stage is the least when the block is as square as the grid allows
    const int xcd = L & 7, idx = L >> 3, bm = tiles_m >> 1;
    tn_i = (xcd >> 1) * (tiles_n >> 2) + idx / bm;
    tm_i = (xcd & 1) * bm + idx % bm;
  } else {
    if (total % 8 == 0) L = (L & 7) * (total >> 3) + (L >> 3);
    tn_i = L / tiles_m;
    tm_i = L % tiles_m;
  }
  const int n0 = tn_i * 256, m0 = tm_i * 256;
  const int wg = words(G);

  // What this lane fetches (byte offsets; 32 bits: the launcher bounds the operands).
  // Rows past N or M are clamped to the last one; their results are never stored.
  uint32_t wo[WI], xo[XI];
#pragma unroll
  for (int i = 0; i < WI; ++i) {
    const int n = n0 + (wave + WAVES * i) * 32 + (lane >> 1);
    wo[i] = (uint32_t)(n < N ? n : N - 1) * (uint32_t)(K >> 1) + (lane & 1) * 16;
  }
#pragma unroll
  for (int i = 0; i < XI; ++i) {
    const int R = (wave + WAVES * i) * 8 + (lane >> 3), m = m0 + R;
    xo[i] = (uint32_t)(m < M ? m : M - 1) * (uint32_t)(K * 2) + (((lane & 7) ^ t2_x_key(R)) * 16);
  }
  // per stage: the dword that holds the scale(s) of W row 64 wave + lane, and (ASYM) the
  // word that holds its zero-point
  const uint32_t sn = (uint32_t)(n0 + wave * 64 + lane < N ? n0 + wave * 64 + lane : N - 1);
  const uint32_t sc_base = sn * (uint32_t)G, zw_base = sn * (uint32_t)wg;
  const char* wqb = (const char*)wq;
  const char* xb = (const char*)x;
  const int stages = K >> 6;

  // The loads are asm so that the compiler neither tracks them (it would wait for all of
  // them before any LDS read) nor moves LDS reads across them; the vmcnt waits below are
  // by hand.  M0 carries the wave-uniform LDS address.
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
  const uint32_t lds0 = (uint32_t)(uintptr_t)(lds_ptr)t2_lds;
  // group of the stage's first k (W4)
  auto group_of = [&](uint32_t d) { return GS32 ? 2u * d : (d * 64u) / (uint32_t)gs; };
  // Load instruction `part` (0 .. LOADS - 1) of stage d into the buffer at byte offset buf.
  // A stage past the last is fetched from the last one and never used.
  auto request_part = [&](int d, uint32_t buf, int part) {
    const uint32_t dd = (uint32_t)(d < stages ? d : stages - 1);
    const uint32_t st = lds0 + buf;
    if (part < WI) {  // the stage's offset goes into the scalar base: no vector arithmetic
      dma16(wqb + dd * 32u, wo[part], st + (wave + WAVES * part) * 1024);
    } else if (part < WI + XI) {
      const int i = part - WI;
      dma16(xb + dd * 128u, xo[i], st + T2_W_BYTES + (wave + WAVES * i) * 1024);
    } else if (part == WI + XI) {
      // MXFP4: the dword around the stage's two E8M0 bytes; gs = 32: the dword of its two
      // scales; else the dword around its one scale
      const uint32_t off = MX ? ((sc_base + 2u * dd) & ~3u)
                              : GS32 ? (sc_base + 2u * dd) * 2u : ((sc_base + group_of(dd)) >> 1) * 4u;
      dma4(scales, off, st + T2_TILE + wave * 256);
    } else {
      dma4(zeros, (zw_base + (group_of(dd) >> 3)) * 4u, st + T2_TILE + 1024 + wave * 256);
    }
  };

  // this lane's rows of the two W tiles of its wave, and where their first scale sits in
  // the dword fetched around it
  const int wrow0 = wave * 64 + r;
  uint32_t par[NI];
#pragma unroll
  for (int i = 0; i < NI; ++i) {
    const int n = n0 + wrow0 + 32 * i;
    par[i] = ((uint32_t)(n < N ? n : N - 1) * (uint32_t)G) & (MX ? 3u : 1u);
  }
  uint32_t mask = 0x00F0000Fu, magic = 0x54006400u;
  asm volatile("" : "+s"(mask));   // opaque: otherwise they come back as literals of two
  asm volatile("" : "+v"(magic));  // separate instructions

  u4 xv[2][MJ];  // X operands of the step in hand and of the next: [m tile]
  u4 wv[NI];     // the stage's packed words: [n tile], word = step
  u4 av[2][NI];  // expanded W operands (as four packed-half registers) of the step in hand and of the next
  uint32_t sc[NI], zw[NI];
  h2 cneg[NI], s2v[NI];
  float sf[NI];
  // Where this lane reads inside a stage buffer, worked out once: the X piece of step u in
  // m tile 0 (tile j is 4 KB further), its four words in n tile 0 (tile 1 is 1 KB further).
  uint32_t xoff[4];
#pragma unroll
  for (int u = 0; u < 4; ++u) xoff[u] = T2_W_BYTES + t2_x_at(r, 4 * h + u);
  const uint32_t woff = t2_w_at(wrow0, h), scoff = T2_TILE + wrow0 * 4;
  auto read_x = [&](u4* dst, uint32_t buf, int u, int j0, int j1) {  // m tiles j0 .. j1 - 1 of step u
    const uint8_t* p = t2_lds + (buf + xoff[u]);
#pragma unroll
    for (int j = j0; j < j1; ++j) dst[j] = *(const u4*)(p + j * 4096);
  };
  auto read_w = [&](uint32_t buf) {
    const uint8_t* p = t2_lds + (buf + woff);
#pragma unroll
    for (int i = 0; i < NI; ++i) wv[i] = *(const u4*)(p + i * 1024);
  };
  auto read_sc = [&](uint32_t buf) {
    const uint8_t* p = t2_lds + (buf + scoff);
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      sc[i] = *(const uint32_t*)(p + i * 128);
      if (ASYM) zw[i] = *(const uint32_t*)(p + 1024 + i * 128);
    }
  };
  auto set_group = [&](int d) {
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      if constexpr (MX) {  // block 2 d + h of the row
        sf[i] = mx_scale((sc[i] >> (8 * (((par[i] + 2u * d) & 3u) + h))) & 0xFFu);
      } else {
        const uint32_t g = group_of((uint32_t)d) + (GS32 ? h : 0);
        const bool hi = GS32 ? h != 0 : ((par[i] + g) & 1u) != 0;
        s2v[i] = splat_bits(hi ? (sc[i] >> 16) : (sc[i] & 0xFFFFu));
        const uint32_t z = ASYM ? ((zw[i] >> (4 * (g & 7))) & 0xFu) : 8u;
        cneg[i] = as_h2(0xD400E400u | (z << 20) | z);
      }
    }
  };
  // register e (k 2 e, 2 e + 1 of the word) of n tile i's operand for step u
  auto expand_reg = [&](u4* dst, int u, int i, int e) {
    const uint32_t w = wv[i][u];
    if constexpr (MX) {
      h2 v = e == 0 ? __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, sf[i], 0)
           : e == 1 ? __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, sf[i], 1)
           : e == 2 ? __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, sf[i], 2)
                    : __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, sf[i], 3);
      dst[i][e] = as_u32(v);
    } else {
      // byte e to bytes 0 and 2; the low nibble into the significand of 1024.0, the high
      // one into that of 64.0; minus (1024 + z), (64 + z): exact; times the scale: one rounding
      const uint32_t p = __builtin_amdgcn_perm(0u, w, 0x0c000c00u | (uint32_t)(e << 16) | (uint32_t)e);
      const uint32_t v = (p & mask) | magic;
      dst[i][e] = as_u32((as_h2(v) + cneg[i]) * s2v[i]);
    }
  };
  auto expand = [&](u4* dst, int u) {
#pragma unroll
    for (int i = 0; i < NI; ++i)
#pragma unroll
      for (int e = 0; e < 4; ++e) expand_reg(dst, u, i, e);
  };

  // The same in four phases over NR registers at once (e0 .. e0 + NR - 1 of n tile i), one
  // phase per MFMA: the four instructions of a register depend on each other, and a wave
  // that issues them back to back waits out each one's latency.  t: the values in between.
  auto expand_phase = [&](int ph, u4* dst, uint32_t* t, int u, int i, int e0, int nr) {
    const uint32_t w = wv[i][u];
#pragma unroll
    for (int q = 0; q < nr; ++q) {
      const int e = e0 + q;
      if constexpr (MX) {
        if (ph == q % 4) expand_reg(dst, u, i, e);
      } else {
        if (ph == 0) t[q] = __builtin_amdgcn_perm(0u, w, 0x0c000c00u | (uint32_t)(e << 16) | (uint32_t)e);
        if (ph == 1) t[q] = (t[q] & mask) | magic;
        if (ph == 2) t[q] = as_u32(as_h2(t[q]) + cneg[i]);
        if (ph == 3) dst[i][e] = as_u32(as_h2(t[q]) * s2v[i]);
      }
    }
  };

  f16v acc[NI][MJ];
#pragma unroll
  for (int i = 0; i < NI; ++i)
#pragma unroll
    for (int j = 0; j < MJ; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  // A stage is sixteen chunks of four MFMAs.  A chunk issues at most one load instruction,
  // reads two tiles of X and expands two operand registers of the next step, one of the four
  // dependent instructions of each under each MFMA.  The barrier at the start of step 3 of
  // stage d frees that stage's buffer; the sixteen chunks from there (step 3 of stage d,
  // steps 0 .. 2 of stage d + 1) request stage d + 3 into it.  b0, b1, b2: byte offsets of
  // the buffers of stages d, d + 1, d + 2 (d + 3 takes b0 again).
  uint32_t b0 = 0, b1 = T2_STAGE, b2 = 2 * T2_STAGE;
#pragma unroll
  for (int part = 0; part < LOADS; ++part) request_part(0, b0, part);
#pragma unroll
  for (int part = 0; part < LOADS; ++part) request_part(1, b1, part);
#pragma unroll
  for (int part = 0; part < CH; ++part) request_part(2, b2, part);
  __builtin_amdgcn_s_waitcnt(t2_waitcnt_vm(LOADS + CH));  // stage 0 has landed
  __syncthreads();
  read_x(xv[0], b0, 0, 0, MJ);
  read_w(b0);
  read_sc(b0);
  set_group(0);
  expand(av[0], 0);
  auto mfma1 = [&](int cur, int c, int k) {  // MFMA 4 c + k of a step
    const int i = (4 * c + k) / MJ, j = (4 * c + k) % MJ;
    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(
        __builtin_bit_cast(h8, av[cur][i]), __builtin_bit_cast(h8, xv[cur][j]), acc[i][j], 0, 0, 0);
  };
  constexpr int RPC = 8 / CH, XPC = MJ / CH;  // operand registers expanded, X tiles read per chunk
  uint32_t tmp[4];
#pragma unroll 1
  for (int d = 0; d < stages; ++d) {
#pragma unroll
    for (int u = 0; u < 3; ++u) {
      const int cur = u & 1, nxt = cur ^ 1;
#pragma unroll
      for (int c = 0; c < CH; ++c) {
        // operands of step u + 1: XPC tiles of X read and RPC registers expanded per chunk
        if (CH + CH * u + c < LOADS) request_part(d + 2, b2, CH + CH * u + c);
        __builtin_amdgcn_sched_barrier(0);
        read_x(xv[nxt], b0, u + 1, XPC * c, XPC * c + XPC);
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          expand_phase(k, av[nxt], tmp, u + 1, (RPC * c) >> 2, (RPC * c) & 3, RPC);
          mfma1(cur, c, k);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }
    // Step 3.  Every LDS read of stage d has been issued (the X operands of this step during
    // step 2, the words at the stage's start): once all waves are here its buffer can take
    // stage d + 3, and stage d + 1 has landed for everyone (outstanding: all of stage d + 2).
    __builtin_amdgcn_s_waitcnt(t2_waitcnt_vm(LOADS));
    __syncthreads();
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      request_part(d + 3, b0, c);
      __builtin_amdgcn_sched_barrier(0);
      if (c == 0) {  // operands of step 0 of stage d + 1: the words, their scales, half of X
        read_w(b1);
        read_sc(b1);
        read_x(xv[0], b1, 0, 0, 4);
      } else if (c == 1) {
        read_x(xv[0], b1, 0, 4, 8);
        set_group(d + 1);
      }
      if (c < 2) {
#pragma unroll
        for (int k = 0; k < 4; ++k) mfma1(1, c, k);
        if (c == 0) __builtin_amdgcn_sched_group_barrier(0x100, 4 + NI + NI * (ASYM ? 2 : 1), 0);
        if (c == 1) __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          if (c > 0) __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
      } else {
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          expand_phase(k, av[0], tmp, 0, c - 2, 0, 4);
          mfma1(1, c, k);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }
    const uint32_t first = b0;
    b0 = b1;
    b1 = b2;
    b2 = first;
  }
  __builtin_amdgcn_s_waitcnt(t2_waitcnt_vm(0));  // nothing may still be writing LDS at exit

  // A lane holds, of each 32 x 32 tile, n = 8 q + 4 h + e for m = tile row r.  The tiles go
  // through LDS (free by now) so that every store instruction writes eight whole 128-byte
  // lines: a wave lays its 256 (m) x 64 (n) block out in rows of 144 bytes and reads it
  // back 16 bytes a lane.  Rows past M and columns past N stay in LDS.
  __syncthreads();  // no wave reads a stage buffer any more, no load is landing in one
  uint8_t* mine = t2_lds + wave * (32 * MJ * T2_C_PITCH);
#pragma unroll
  for (int j = 0; j < MJ; ++j) {
    // the sums of an m tile leave the accumulator registers only when its turn comes (256
    // of them copied out at once would not fit beside everything else)
    asm volatile("" : "+a"(acc[0][j]), "+a"(acc[1][j]));
#pragma unroll
    for (int i = 0; i < NI; ++i)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        h4 out;
#pragma unroll
        for (int e = 0; e < 4; ++e) out[e] = (_Float16)acc[i][j][4 * q + e];
        *(h4*)(mine + (j * 32 + r) * T2_C_PITCH + i * 64 + q * 16 + h * 8) = out;
      }
    __builtin_amdgcn_sched_barrier(0);
  }
  const bool lines = (N & 7) == 0 && ((uintptr_t)c & 15) == 0;  // 16-byte pieces are aligned
  const int nn = n0 + wave * 64 + (lane & 7) * 8;
#pragma unroll 4
  for (int it = 0; it < 32 * MJ / 8; ++it) {
    const int row = it * 8 + (lane >> 3), m = m0 + row;
    if (m >= M || nn >= N) continue;
    const u4 v = *(const u4*)(mine + row * T2_C_PITCH + (lane & 7) * 16);
    w4_half* dst = c + (size_t)m * N + nn;
    if (lines && nn + 8 <= N) {
      *(u4*)dst = v;
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e)
        if (nn + e < N) dst[e] = (w4_half)(v[e >> 1] >> (16 * (e & 1)));
    }
  }
}

template <int FMT, bool GS32>
hipError_t launch(const WView& v, const w4_half* x, w4_half* c, int M, hipStream_t s, int tiles_n,
                  int tiles_m) {
  // more than 64 KB of LDS has to be granted per device, once
  static std::atomic<bool> granted[64] = {};
  int dev = 0;
  if (hipError_t e = hipGetDevice(&dev); e != hipSuccess) return e;
  if (dev < 0 || dev >= 64 || !granted[dev]) {
    const hipError_t e = hipFuncSetAttribute((const void*)w4_tile256_kernel<FMT, GS32>,
                                             hipFuncAttributeMaxDynamicSharedMemorySize, T2_LDS);
    if (e != hipSuccess) return e;
    if (dev >= 0 && dev < 64) granted[dev] = true;
  }
  w4_tile256_kernel<FMT, GS32><<<dim3((unsigned)(tiles_n * tiles_m)), dim3(T2_THREADS), T2_LDS, s>>>(
      v.q, v.scales, v.zeros, x, c, v.N, v.K, v.mx ? v.B : v.G, v.gs, M, tiles_n, tiles_m);
  return hipGetLastError();
}

}  // namespace

// For the caller that has already checked what both tile kernels need (K a multiple of
// 128, gs 32, 64 or a multiple of 128, operands under 4 GiB, alignments): takes the call
// when 256 x 256 tiles cover the problem in at most half the rounds that 128 x 256 tiles
// need on `cus` compute units (one workgroup each), and launches nothing otherwise.
bool try_tile256(const WView& v, const w4_half* x, w4_half* c, int M, hipStream_t s, int cus,
                 hipError_t* err) {
  const long long n256 = (v.N + 255) / 256, m256 = (M + 255) / 256, m128 = (M + 127) / 128;
  const long long r256 = (n256 * m256 + cus - 1) / cus, r128 = (n256 * m128 + cus - 1) / cus;
  if (2 * r256 > r128 || n256 * m256 > 0x7FFFFFFFLL) return false;
  const int tn = (int)n256, tm = (int)m256;
  if (v.mx) *err = launch<2, false>(v, x, c, M, s, tn, tm);
  else if (v.symmetric) *err = v.gs == 32 ? launch<0, true>(v, x, c, M, s, tn, tm) : launch<0, false>(v, x, c, M, s, tn, tm);
  else *err = v.gs == 32 ? launch<1, true>(v, x, c, M, s, tn, tm) : launch<1, false>(v, x, c, M, s, tn, tm);
  return true;
}

}  // namespace w4k
