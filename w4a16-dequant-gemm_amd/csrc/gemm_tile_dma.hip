// Large-M W4A16 GEMM whose operands reach LDS without passing through registers:
// c[M,N] = X[M,K] * dequant(W)[N,K]^T for W4 weights with FP16 group scales and
// optional 4-bit zero-points (mma.cuh:63-230 is the reference's tensor-core kernel:
// it expands each chunk of W to FP16 in shared memory once per block).
//
// Here the packed words themselves are what sits in LDS -- a quarter of the bytes
// of the expanded tile -- and every wave expands the words of its own MFMA
// operands in registers, straight into the operand layout:
//   * global_load_lds_dwordx4 moves both operand tiles global -> LDS (no staging
//     registers, no ds_write); a stage is 128 k: 64 bytes of a W row, 256 bytes of
//     an X row; three stages of 50 KB; one barrier per stage.
//   * v_mfma_f32_32x32x16_f16: lane l brings row l%32 and eight consecutive k.
//     Which eight is free as long as both operands agree, so of a 64-k half lane
//     half h = l/32 takes k 32h + 8j .. + 7 in MFMA j: its four W words are one
//     16-byte LDS read, its X operand is 16-byte piece 4h + j of the row's half.
//   * a word becomes four packed-half registers in natural k order with
//     v_perm_b32 (byte i to bytes 0 and 2), one mask-and-or that plants the low
//     nibble in the significand of 1024.0 and the high nibble in that of 64.0
//     (whose unit in the last place is 1/16), one packed add of -(1024 + z),
//     -(64 + z) and one packed multiply by the scale: q - z is exact and the
//     product is rounded once, so the operand is bit for bit the FP16 weight the
//     one dequant step returns (pack.hpp:58-60).
// The accumulation is FP32 in the instruction; the output is rounded to FP16 once.
#include <atomic>

#include "dq.cuh"
#include "kernels.h"

namespace w4k {
namespace {

typedef float f16v __attribute__((ext_vector_type(16)));
typedef __attribute__((address_space(3))) void* lds_ptr;

// rows of W (TN: 256 or 128) and of X (TM: 128, 64 or 32) per workgroup are template parameters
constexpr int TD_WAVES = 4, TD_THREADS = 64 * TD_WAVES;  // a wave: 64 rows of W x all 128 of X
constexpr int TD_STAGES = 3;
// a stage: TN rows of W (64 bytes each), TM rows of X (256 bytes each), two scale dwords and a
// zero-point word per W row
constexpr int td_tile(int tm, int tn) { return tn * 64 + tm * 256; }
constexpr int td_stage(int tm, int tn) { return td_tile(tm, tn) + 3 * tn * 4; }
constexpr int td_lds_bytes(int tm, int tn) { return TD_STAGES * td_stage(tm, tn); }

// s_waitcnt vmcnt(N) alone (gfx9 encoding: vmcnt in [3:0] and [15:14])
constexpr int waitcnt_vm(int n) { return (n & 0xF) | ((n >> 4) << 14) | 0x0F70; }

extern __shared__ __attribute__((aligned(16))) uint8_t td_lds[];

// Position of 16-byte piece p of row R.  A load instruction writes lane l's 16
// bytes at 16 l, so the rows of one instruction are contiguous (16 rows of W, 4 of
// X) and the piece a lane fetches is chosen so that the rows one ds_read_b128
// touches (8 or 16 consecutive ones, same p) fall on distinct 16-byte bank groups.
__device__ __forceinline__ int w_key(int R) { return ((R >> 1) ^ (R >> 3)) & 3; }
__device__ __forceinline__ int w_at(int R, int p) {
  return (R >> 4) * 1024 + ((R & 15) * 4 + (p ^ w_key(R))) * 16;
}
__device__ __forceinline__ int x_at(int R, int p) {
  return (R >> 2) * 1024 + ((R & 3) * 16 + (p ^ (R & 15))) * 16;
}

// Eight codes of a packed word -> eight FP16 weights in k order (as an MFMA operand).
// cneg: packed {-(1024 + z), -(64 + z)}; s2: the group scale in both halves.
// mask, magic: 0x00F0000F and 0x54006400 held in registers (the three-operand
// and-or takes no literal).
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

// One wave per SIMD, so the three pipes have to overlap inside a wave: a stage is
// eight steps of 16 k (8 MFMAs each); during the MFMAs of step u the wave reads the
// X operands of step u + 1 from LDS and expands its W words, in program order
// between the MFMAs.
//
// HOOK: the workgroups of the first m tile also write the expanded weights to
// w_out (mma.cuh:147-159: the reference's dequant hook), from the operand
// registers the MFMAs consume.
//
// FMT: 0 W4 symmetric, 1 W4 with zero-points, 2 MXFP4.  GSM says how the groups
// lie in a 128-k stage: 0 one group (gs a multiple of 128), 1 two (gs = 64), 2 four
// (gs = 32, and the 32-blocks of MXFP4).  A lane's share of a 64-k half is 32
// consecutive k, so even then it has one scale per half.  G: scales per row.
// TM: rows of X per workgroup, 128, 64 or 32 (a wave: 64 rows of W x all TM of X).  The
// smaller tile halves a workgroup's walk over K when the grid of the larger one
// would leave most of the chip idle.
// TN: rows of W per workgroup, 256 or 128 (a wave: TN / 4 of them = NI tiles of 32).
// KG: sets of four waves per workgroup.  With two, each set walks one half of the K / 128
// stages through stage buffers of its own (two waves per SIMD, whose instruction streams
// interleave) and the second set's sums are added to the first set's at the end, through
// LDS: on the thin grids of the small tiles a workgroup's stages are a chain of 0.6 us
// each whatever they hold, and this halves the chain.  split_at: the hooked kernel, which
// always has one set, starts a second accumulator at that stage and adds the two at the
// end, so that it returns the bytes of the two-set kernel (no split: a stage past the last).
template <int FMT, int GSM, bool HOOK, int TM, int TN, int KG>
__global__ __launch_bounds__(TD_THREADS * KG) void w4_tile_dma_kernel(
    const uint32_t* __restrict__ wq, const void* __restrict__ scales,
    const uint32_t* __restrict__ zeros, const w4_half* __restrict__ x, w4_half* __restrict__ c,
    w4_half* __restrict__ w_out, int N, int K, int G, int gs, int M, int tiles_n, int tiles_m,
    int split_at) {
  constexpr bool ASYM = FMT == 1, MX = FMT == 2;
  constexpr int NSC = (!MX && GSM == 2) ? 2 : 1;           // scale dwords per row and stage
  constexpr int TD_TM = TM, MJ = TM / 32;                  // 32-row tiles of X per wave
  constexpr int TD_TN = TN, NI = TN / 128;                 // 32-row tiles of W per wave
  constexpr int TD_W_BYTES = TN * 64;
  constexpr int TD_WI = TD_W_BYTES / 1024 / TD_WAVES;      // 1 KB load instructions of W per wave
  constexpr int TD_TILE = td_tile(TM, TN), TD_STAGE = td_stage(TM, TN);
  constexpr int TD_XI = TM * 256 / 1024 / TD_WAVES;        // 1 KB load instructions of X per wave
  constexpr int LOADS = TD_WI + TD_XI + NSC + (ASYM ? 1 : 0);  // load instructions per wave and stage
  constexpr bool PHASED = NI * MJ >= 4;  // a step has the four MFMAs that the phases of an expansion go under
  const int t = threadIdx.x, lane = t & 63;
  const int wave_all = __builtin_amdgcn_readfirstlane(t >> 6);  // in an SGPR: LDS addresses go to M0
  const int wave = KG == 2 ? (wave_all & 3) : wave_all;        // within its set of four
  const int grp = KG == 2 ? (wave_all >> 2) : 0;               // the set
  const int r = lane & 31, h = lane >> 5;
  // Consecutive workgroup ids land on different XCDs (each with its own L2): give
  // each XCD a contiguous run of the tile order, m fastest, so that its
  // workgroups share a few W tiles and walk X.
  int L = blockIdx.x;
  const int total = tiles_n * tiles_m;
  if (total % 8 == 0) L = (L & 7) * (total >> 3) + (L >> 3);
  const int n0 = (L / tiles_m) * TD_TN, m0 = (L % tiles_m) * TD_TM;
  const int wg = words(G);

  // What this lane fetches (byte offsets; 32 bits: the launcher bounds the operands).
  // Rows past N or M are clamped to the last one; their results are never stored.
  uint32_t wo[TD_WI], xo[TD_XI];
#pragma unroll
  for (int i = 0; i < TD_WI; ++i) {
    const int R = (wave + TD_WAVES * i) * 16 + (lane >> 2), n = n0 + R;
    wo[i] = (uint32_t)(n < N ? n : N - 1) * (uint32_t)(K >> 1) + (((lane & 3) ^ w_key(R)) * 16);
  }
#pragma unroll
  for (int i = 0; i < TD_XI; ++i) {
    const int R = (wave + TD_WAVES * i) * 4 + (lane >> 4), m = m0 + R;
    xo[i] = (uint32_t)(m < M ? m : M - 1) * (uint32_t)(K * 2) + (((lane & 15) ^ (R & 15)) * 16);
  }
  // per stage: the dword that holds the group scale of W row 64 wave + lane, and
  // (ASYM) that row's zero-point word
  // (TN = 128: waves 2 and 3 repeat the fetches of waves 0 and 1, which keeps the count of
  // load instructions the same for every wave)
  const int srow = (NI == 2 ? wave : (wave & 1)) * 64 + lane;
  const uint32_t sn = (uint32_t)(n0 + srow < N ? n0 + srow : N - 1);
  const uint32_t sc_base = sn * (uint32_t)G, zw_base = sn * (uint32_t)wg;
  const char* wqb = (const char*)wq;
  const char* xb = (const char*)x;

  const int stages = K >> 7;
  // this set's stages: d_first .. d_first + per_set - 1, those below `stages` (both sets run
  // per_set iterations so that they meet at every barrier; a stage past the end is fetched
  // from the last one and not multiplied)
  const int per_set = (stages + KG - 1) / KG;
  const int d_first = grp * per_set;
  const int d_end = min(d_first + per_set, stages) > d_first ? min(d_first + per_set, stages) : d_first + 1;
  // The loads are asm so that the compiler neither tracks them (it would wait for
  // all of them before any LDS read) nor moves LDS reads across them; the vmcnt
  // waits below are by hand.  M0 carries the wave-uniform LDS address.
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
  const uint32_t lds0 = (uint32_t)(uintptr_t)(lds_ptr)td_lds;
  // Load instruction `part` (0 .. LOADS - 1) of stage d: a wave issues them two at
  // a time between the MFMAs of successive steps -- thirteen in a row would hold up
  // its one instruction stream for as long as four steps take.
  auto request_part = [&](int d, uint32_t buf, int part) {  // buf: byte offset of the stage's buffer
    const uint32_t dd = (uint32_t)(d < d_end ? d : d_end - 1);  // past the set's end: valid, never used
    const uint32_t st = lds0 + buf;
    if (part < TD_WI) {  // the stage's offset goes into the scalar base: no vector arithmetic
      dma16(wqb + dd * 64u, wo[part], st + (wave + TD_WAVES * part) * 1024);
    } else if (part < TD_WI + TD_XI) {
      const int i = part - TD_WI;
      dma16(xb + dd * 256u, xo[i], st + TD_W_BYTES + (wave + TD_WAVES * i) * 1024);
    } else {
      // the stage's scales of this wave's row 64 wave + lane: the dword with the one
      // FP16 scale (GSM 0), the dword of its two (GSM 1), the two dwords of its four
      // (GSM 2), the four E8M0 bytes (MXFP4); then the zero-point word
      const int k = part - TD_WI - TD_XI;
      const uint32_t g = MX ? dd * 4u : GSM == 0 ? (dd * 128u) / (uint32_t)gs : dd * (2u * GSM);
      if (k < NSC) {
        const uint32_t off = MX ? sc_base + g : GSM == 0 ? ((sc_base + g) >> 1) * 4u
                                                        : (sc_base + g) * 2u + 4u * k;
        dma4(scales, off, st + TD_TILE + k * (TD_TN * 4) + (NI == 2 ? wave : (wave & 1)) * 256);
      } else {
        dma4(zeros, (zw_base + (g >> 3)) * 4u,
             st + TD_TILE + 2 * (TD_TN * 4) + (NI == 2 ? wave : (wave & 1)) * 256);
      }
    }
  };
  auto request = [&](int d, uint32_t buf) {
#pragma unroll
    for (int part = 0; part < LOADS; ++part) request_part(d, buf, part);
  };

  // this lane's rows of the two W tiles of its wave; the parity of their first
  // scale index says which half of the fetched dword is theirs
  int wrow[NI];
  uint32_t par[NI];
#pragma unroll
  for (int i = 0; i < NI; ++i) {
    wrow[i] = wave * (32 * NI) + i * 32 + r;
    const int n = n0 + wrow[i];
    par[i] = ((uint32_t)(n < N ? n : N - 1) * (uint32_t)G) & 1u;
  }
  const bool hook = HOOK && m0 == 0;
  uint32_t mask = 0x00F0000Fu, magic = 0x54006400u;
  asm volatile("" : "+s"(mask));   // opaque: otherwise they come back as literals of two
  asm volatile("" : "+v"(magic));  // separate instructions

  u4 xv[2][MJ];           // X operands of the step in hand and of the next: [m tile]
  u4 wv[2][NI];           // packed words of the two 64-k halves: [half][n tile], word = step % 4
  u4 av[2][NI];           // expanded W operands (four packed-half registers) of the step in hand and of the next
  uint32_t sc[NI][NSC], zw[NI];  // the stage's scale dwords and zero-point word per n tile
  // what expansion needs, per [half][n tile]: -(1024 + z), -(64 + z) and the scale in
  // both halves of a register (MXFP4: the scale as a float)
  h2 cneg[2][NI], s2v[2][NI];
  float sf[2][NI];
  // Where this lane reads inside a stage buffer, worked out once: the X piece of
  // step u in m tile 0 (tile j is 8 KB further), its four words of half s2 in n tile
  // 0 (tile 1 is 2 KB further), its scale dword.  A read is then one add of the
  // buffer's offset and an immediate.
  uint32_t xoff[8], woff[2];
#pragma unroll
  for (int u = 0; u < 8; ++u) xoff[u] = TD_W_BYTES + x_at(r, 8 * (u >> 2) + 4 * h + (u & 3));
#pragma unroll
  for (int s2 = 0; s2 < 2; ++s2) woff[s2] = w_at(wrow[0], 2 * s2 + h);
  const uint32_t scoff = TD_TILE + wrow[0] * 4;
  auto read_x = [&](u4* dst, uint32_t buf, int u) {  // step u = half u/4, MFMA u%4
    const uint8_t* p = td_lds + (buf + xoff[u]);
#pragma unroll
    for (int j = 0; j < MJ; ++j) dst[j] = *(const u4*)(p + j * 8192);
  };
  auto read_w = [&](u4* dst, uint32_t buf, int s2) {
    const uint8_t* p = td_lds + (buf + woff[s2]);
#pragma unroll
    for (int i = 0; i < NI; ++i) dst[i] = *(const u4*)(p + i * 2048);
  };
  auto read_sc = [&](uint32_t buf) {
    const uint8_t* p = td_lds + (buf + scoff);
#pragma unroll
    for (int i = 0; i < NI; ++i) {
#pragma unroll
      for (int k = 0; k < NSC; ++k) sc[i][k] = *(const uint32_t*)(p + k * (TD_TN * 4) + i * 128);
      if (ASYM) zw[i] = *(const uint32_t*)(p + 2 * (TD_TN * 4) + i * 128);
    }
  };
  auto set_group = [&](int d) {
#pragma unroll
    for (int s2 = 0; s2 < 2; ++s2)
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        if constexpr (MX) {  // block 4 d + 2 s2 + h of the row
          sf[s2][i] = mx_scale((sc[i][0] >> (8 * (2 * s2 + h))) & 0xFFu);
        } else {
          uint32_t g, s16;
          if constexpr (GSM == 0) {
            g = ((uint32_t)d * 128u) / (uint32_t)gs;
            s16 = ((par[i] + g) & 1u) ? (sc[i][0] >> 16) : (sc[i][0] & 0xFFFFu);
          } else if constexpr (GSM == 1) {
            g = 2u * d + s2;
            s16 = s2 ? (sc[i][0] >> 16) : (sc[i][0] & 0xFFFFu);
          } else {
            g = 4u * d + 2 * s2 + h;
            s16 = h ? (sc[i][s2] >> 16) : (sc[i][s2] & 0xFFFFu);
          }
          s2v[s2][i] = splat_bits(s16);
          const uint32_t z = ASYM ? ((zw[i] >> (4 * (g & 7))) & 0xFu) : 8u;
          cneg[s2][i] = as_h2(0xD400E400u | (z << 20) | z);
        }
      }
  };
  auto hook_store = [&](const u4* src, int d, int u, int i) {
    if (HOOK && hook && d < stages && n0 + wrow[i] < N)
      *(u4*)(w_out + (size_t)(n0 + wrow[i]) * K + d * 128 + (u >> 2) * 64 + h * 32 + (u & 3) * 8) = src[i];
  };
  auto expand = [&](u4* dst, int d, int u) {
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      if constexpr (MX) {
        h2 n4[4];
        dq_mx(wv[u >> 2][i][u & 3], sf[u >> 2][i], n4);
        dst[i] = u4{as_u32(n4[0]), as_u32(n4[1]), as_u32(n4[2]), as_u32(n4[3])};
      } else {
        dst[i] = __builtin_bit_cast(
            u4, expand_word(wv[u >> 2][i][u & 3], cneg[u >> 2][i], s2v[u >> 2][i], mask, magic));
      }
      hook_store(dst, d, u, i);
    }
  };
  // The same in four phases over the registers e0 .. e0 + nr - 1 of n tile i, one phase per
  // MFMA: the four instructions of a register depend on each other, and a wave that issues
  // them back to back waits out each one's latency.  t: the values in between.
  auto expand_phase = [&](int ph, u4* dst, uint32_t* t, int u, int i, int e0, int nr) {
    const uint32_t w = wv[u >> 2][i][u & 3];
#pragma unroll
    for (int q = 0; q < nr; ++q) {
      const int e = e0 + q;
      if constexpr (MX) {
        const float sc_f = sf[u >> 2][i];
        if (ph == q % 4)
          dst[i][e] = as_u32(e == 0   ? __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, sc_f, 0)
                             : e == 1 ? __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, sc_f, 1)
                             : e == 2 ? __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, sc_f, 2)
                                      : __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, sc_f, 3));
      } else {
        if (ph == 0) t[q] = __builtin_amdgcn_perm(0u, w, 0x0c000c00u | (uint32_t)(e << 16) | (uint32_t)e);
        if (ph == 1) t[q] = (t[q] & mask) | magic;
        if (ph == 2) t[q] = as_u32(as_h2(t[q]) + cneg[u >> 2][i]);
        if (ph == 3) dst[i][e] = as_u32(as_h2(t[q]) * s2v[u >> 2][i]);
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

  // Stage d + 2 is requested in pieces from step 7 of stage d - 1 (when the barrier
  // there has freed its buffer) to step 6 of stage d.  b0, b1, b2: byte offsets of
  // the buffers of stages d, d + 1, d + 2 (d + 3 takes b0 again).
  const uint32_t set_base = grp * (TD_STAGES * TD_STAGE);
  uint32_t b0 = set_base, b1 = set_base + TD_STAGE, b2 = set_base + 2 * TD_STAGE;
  request(d_first, b0);
  request(d_first + 1, b1);
  request_part(d_first + 2, b2, 0);
  request_part(d_first + 2, b2, 1);
  __builtin_amdgcn_s_waitcnt(waitcnt_vm(LOADS + 2));  // stage 0 has landed
  __syncthreads();
  read_x(xv[0], b0, 0);
  read_w(wv[0], b0, 0);
  read_sc(b0);
  set_group(d_first);
  expand(av[0], d_first, 0);
  [[maybe_unused]] f16v acc_first[HOOK ? NI : 1][HOOK ? MJ : 1];
#pragma unroll 1
  for (int it = 0; it < per_set; ++it) {
    const int d = d_first + it;
    if constexpr (HOOK) {
      if (d == split_at) {  // what the second set of waves of the unhooked kernel starts with
#pragma unroll
        for (int i = 0; i < NI; ++i)
#pragma unroll
          for (int j = 0; j < MJ; ++j) {
            acc_first[i][j] = acc[i][j];
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
          }
      }
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      if (u == 7) {
        // every LDS read of stage d has been issued (the X operands of step 7 during
        // step 6): once all waves are here its buffer can take stage d + 3, and stage
        // d + 1 has landed for everyone (outstanding: all of stage d + 2)
        __builtin_amdgcn_s_waitcnt(waitcnt_vm(LOADS));
        __syncthreads();
        request_part(d + 3, b0, 0);
        request_part(d + 3, b0, 1);
        __builtin_amdgcn_sched_barrier(0);
        read_x(xv[0], b1, 0);
        read_w(wv[0], b1, 0);
        read_sc(b1);
        set_group(d + 1);
        expand(av[0], d + 1, 0);
      } else {
        if (2 * u + 2 < LOADS) request_part(d + 2, b2, 2 * u + 2);
        if (2 * u + 3 < LOADS) request_part(d + 2, b2, 2 * u + 3);
        __builtin_amdgcn_sched_barrier(0);
        read_x(xv[(u + 1) & 1], b0, u + 1);
        if (u == 0) read_w(wv[1], b0, 1);
        if constexpr (!PHASED) expand(av[(u + 1) & 1], d, u + 1);
      }
      constexpr int NM = NI * MJ;  // MFMAs of a step
      auto mfma = [&](int k) {
        const int i = k / MJ, j = k % MJ;
        if (KG == 1 || d < stages)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(
              __builtin_bit_cast(h8, av[u & 1][i]), __builtin_bit_cast(h8, xv[u & 1][j]), acc[i][j], 0, 0, 0);
      };
      bool done = false;
      if constexpr (PHASED) if (u < 7) {
        done = true;
        // the operands of step u + 1, expanded under this step's MFMAs: four MFMAs per group
        // of RPG registers, one phase under each
        constexpr int RPG = 16 * NI / NM;  // registers per group of four MFMAs
        uint32_t tmp[RPG];
#pragma unroll
        for (int k = 0; k < NM; ++k) {
          if constexpr (RPG == 4) {  // a group of four MFMAs per word
            expand_phase(k & 3, av[(u + 1) & 1], tmp, u + 1, k >> 2, 0, 4);
            if ((k & 3) == 3) hook_store(av[(u + 1) & 1], d, u + 1, k >> 2);
          } else {  // four MFMAs in all: both words under them
            static_assert(RPG == 8 && NI == 2, "64 rows of X against two tiles of W");
            expand_phase(k & 3, av[(u + 1) & 1], tmp, u + 1, 0, 0, 4);
            expand_phase(k & 3, av[(u + 1) & 1], tmp + 4, u + 1, 1, 0, 4);
            if ((k & 3) == 3) {
              hook_store(av[(u + 1) & 1], d, u + 1, 0);
              hook_store(av[(u + 1) & 1], d, u + 1, 1);
            }
          }
          mfma(k);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      if (!done) {
#pragma unroll
      for (int k = 0; k < NM; ++k) mfma(k);
      // LDS reads first, then the expansion spread evenly under the MFMAs: a wave
      // can issue about six vector instructions in the shadow of one MFMA
      // vector instructions of a step (16 per word, a few more), shared out over its MFMAs
      constexpr int VPM = (16 * NI + 8 + NM - 1) / NM, VPM0 = VPM + 2;
      constexpr int VPM7 = (16 * NI + 16 + NM / 2) / (NM / 2 + 1);
      if (u == 7) {
        // the words to expand have only just been asked for: the first MFMAs cover that
        __builtin_amdgcn_sched_group_barrier(0x100, NI + MJ + NI * NSC + (ASYM ? NI : 0), 0);
#pragma unroll
        for (int k = 0; k < NM / 2 - 1; ++k) __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
#pragma unroll
        for (int k = 0; k < NM / 2 + 1; ++k) {
          __builtin_amdgcn_sched_group_barrier(0x002, VPM7, 0);
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        }
      } else {
        if (u == 0) __builtin_amdgcn_sched_group_barrier(0x100, MJ + NI, 0);
        else __builtin_amdgcn_sched_group_barrier(0x100, MJ, 0);
#pragma unroll
        for (int k = 0; k < NM; ++k) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          if (u == 0) __builtin_amdgcn_sched_group_barrier(0x002, VPM0, 0);
          else __builtin_amdgcn_sched_group_barrier(0x002, VPM, 0);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
      }
    }
    const uint32_t first = b0;
    b0 = b1;
    b1 = b2;
    b2 = first;
  }
  __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));  // nothing may still be writing LDS at exit
  if constexpr (HOOK) {
    if (split_at < stages) {
#pragma unroll
      for (int i = 0; i < NI; ++i)
#pragma unroll
        for (int j = 0; j < MJ; ++j) acc[i][j] = acc_first[i][j] + acc[i][j];
    }
  }
  if constexpr (KG == 2) {
    // the second set's sums go to the first through LDS (the stage buffers are free once
    // every wave is here): first set + second set, in that order
    __syncthreads();
    float* mine = (float*)td_lds + (size_t)wave * (NI * MJ * 16 * 64);
    if (grp == 1) {
#pragma unroll
      for (int i = 0; i < NI; ++i)
#pragma unroll
        for (int j = 0; j < MJ; ++j)
#pragma unroll
          for (int e = 0; e < 16; ++e) mine[((i * MJ + j) * 16 + e) * 64 + lane] = acc[i][j][e];
    }
    __syncthreads();
    if (grp == 1) return;
#pragma unroll
    for (int i = 0; i < NI; ++i)
#pragma unroll
      for (int j = 0; j < MJ; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][j][e] += mine[((i * MJ + j) * 16 + e) * 64 + lane];
  }

  // A lane holds, of each 32 x 32 tile, n = 8 q + 4 h + e for m = tile row r.  Whole
  // tiles go through LDS (free by now) so that every store instruction writes eight
  // whole 128-byte lines instead of 16 bytes of each of 32: a wave lays its 128 (m)
  // x 64 (n) block out in rows of 144 bytes and reads it back 16 bytes a lane.
  const bool whole = m0 + TD_TM <= M && n0 + TD_TN <= N && (N & 7) == 0 && ((uintptr_t)c & 15) == 0;
  if (whole) {
    constexpr int RB = 64 * NI, PITCH = RB + 16;  // bytes of a row of the wave's block, and its LDS pitch
    constexpr int PP = RB / 16, ROWS = 64 / PP;   // 16-byte pieces per row, rows per store instruction
    __syncthreads();  // no wave reads a stage buffer any more, no load is landing in one
    uint8_t* mine = td_lds + wave * (TD_TM * PITCH);
#pragma unroll
    for (int j = 0; j < MJ; ++j)
#pragma unroll
      for (int i = 0; i < NI; ++i)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          h4 out;
#pragma unroll
          for (int e = 0; e < 4; ++e) out[e] = (_Float16)acc[i][j][4 * q + e];
          *(h4*)(mine + (j * 32 + r) * PITCH + i * 64 + q * 16 + h * 8) = out;
        }
    w4_half* cw = c + (size_t)m0 * N + n0 + wave * (32 * NI);
#pragma unroll
    for (int it = 0; it < TD_TM / ROWS; ++it) {
      const int row = it * ROWS + lane / PP, piece = lane % PP;
      const u4 v = *(const u4*)(mine + row * PITCH + piece * 16);
      *(u4*)(cw + (size_t)row * N + piece * 8) = v;
    }
    return;
  }
#pragma unroll
  for (int j = 0; j < MJ; ++j) {
    const int m = m0 + j * 32 + r;
    if (m >= M) continue;
#pragma unroll
    for (int i = 0; i < NI; ++i)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int nn = n0 + wave * (32 * NI) + i * 32 + 8 * q + 4 * h;
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

template <int FMT, int GSM, bool HOOK, int TM, int TN, int KG = 1>
hipError_t launch(const WView& v, const w4_half* x, w4_half* c, w4_half* w_out, int M,
                  hipStream_t s, int tiles_n, int tiles_m, int split_at) {
  constexpr int TD_LDS = KG * td_lds_bytes(TM, TN);
  static_assert(TD_LDS <= 160 * 1024, "the stage buffers of every set of waves fit LDS");
  // more than 64 KB of LDS has to be granted per device, once
  static std::atomic<bool> granted[64] = {};
  int dev = 0;
  if (hipError_t e = hipGetDevice(&dev); e != hipSuccess) return e;
  if (dev < 0 || dev >= 64 || !granted[dev]) {
    const hipError_t e = hipFuncSetAttribute((const void*)w4_tile_dma_kernel<FMT, GSM, HOOK, TM, TN, KG>,
                                             hipFuncAttributeMaxDynamicSharedMemorySize, TD_LDS);
    if (e != hipSuccess) return e;
    if (dev >= 0 && dev < 64) granted[dev] = true;
  }
  w4_tile_dma_kernel<FMT, GSM, HOOK, TM, TN, KG>
      <<<dim3((unsigned)(tiles_n * tiles_m)), dim3(TD_THREADS * KG), TD_LDS, s>>>(
          v.q, v.scales, v.zeros, x, c, w_out, v.N, v.K, v.mx ? v.B : v.G, v.gs, M, tiles_n,
          tiles_m, split_at);
  return hipGetLastError();
}

// shape: 0 = 128 x 256 (rows of X x rows of W), 1 = 64 x 256, 2 = 64 x 128, 3 = 128 x 128,
// 4 = 32 x 128 (the hooked kernels exist for the first only)
// sets: 2 = the small tiles with two sets of waves (the hooked kernel then splits its sum at
// split_at, the first stage of the second set)
template <int FMT, int GSM>
hipError_t launch_hook(const WView& v, const w4_half* x, w4_half* c, w4_half* w_out, int M,
                       hipStream_t s, int tn, int tm, int shape, int sets, int split_at) {
  if (w_out) return launch<FMT, GSM, true, 128, 256>(v, x, c, w_out, M, s, tn, tm, split_at);
  const int none = v.K;  // more than any stage index
  if (shape == 4 && sets == 2) return launch<FMT, GSM, false, 32, 128, 2>(v, x, c, nullptr, M, s, tn, tm, none);
  if (shape == 2 && sets == 2) return launch<FMT, GSM, false, 64, 128, 2>(v, x, c, nullptr, M, s, tn, tm, none);
  if (shape == 4) return launch<FMT, GSM, false, 32, 128>(v, x, c, nullptr, M, s, tn, tm, none);
  if (shape == 3) return launch<FMT, GSM, false, 128, 128>(v, x, c, nullptr, M, s, tn, tm, none);
  if (shape == 2) return launch<FMT, GSM, false, 64, 128>(v, x, c, nullptr, M, s, tn, tm, none);
  if (shape == 1) return launch<FMT, GSM, false, 64, 256>(v, x, c, nullptr, M, s, tn, tm, none);
  return launch<FMT, GSM, false, 128, 256>(v, x, c, nullptr, M, s, tn, tm, none);
}

template <int FMT>
hipError_t launch_gsm(int gsm, const WView& v, const w4_half* x, w4_half* c, w4_half* w_out,
                      int M, hipStream_t s, int tn, int tm, int shape, int sets, int split_at) {
  if (gsm == 0) return launch_hook<FMT, 0>(v, x, c, w_out, M, s, tn, tm, shape, sets, split_at);
  if (gsm == 1) return launch_hook<FMT, 1>(v, x, c, w_out, M, s, tn, tm, shape, sets, split_at);
  return launch_hook<FMT, 2>(v, x, c, w_out, M, s, tn, tm, shape, sets, split_at);
}

}  // namespace

// Takes MXFP4 weights and W4 weights whose groups tile a 128-k stage (gs 32, 64 or a
// multiple of 128), M >= 65, K a multiple of 128, operands under 4 GiB (32-bit offsets),
// 16-byte aligned rows, scales that can be fetched as aligned dwords, and at least
// eight tiles (measured at N = K = 4096: M = 128, 16 tiles, 44 us against 56 us for
// the register-staged kernel).  Returns false, launching nothing, otherwise.
bool try_tile_dma(const WView& v, const w4_half* x, w4_half* c, int M, hipStream_t s,
                  w4_half* w_out, hipError_t* err) {
  if (v.K % 128 || v.K < 128) return false;
  int gsm = 2;
  if (!v.mx) {
    if (v.gs % 128 == 0) gsm = 0;
    else if (v.gs == 64) gsm = 1;
    else if (v.gs != 32) return false;
  }
  // The smallest of the tile shapes whose grid still fits the chip's 256 compute
  // units in one round: a smaller tile shortens a workgroup's walk over K -- N = K =
  // 4096, M = 512: 45.6 us with 128 x 256 tiles, 38.1 with 64 x 256, 27.0 with 64 x 128;
  // M = 256: 23.7 with 64 x 128 (128 workgroups), 21.8 with 32 x 128 (256).  On such grids a
  // workgroup's K / 128 stages are a chain of 0.6 - 0.7 us each whatever the tile holds.
  // (Hooked
  // and unhooked calls add in the same order whatever the shape: a wave's sums do
  // not depend on how many rows its workgroup holds.)
  const long long n256 = (v.N + 255) / 256, n128 = (v.N + 127) / 128;
  const long long m128 = (M + 127) / 128, m64 = (M + 63) / 64, m32 = (M + 31) / 32;
  // the shape an unhooked call takes; the hooked kernel has 128 x 256 tiles only, but follows
  // the unhooked call's split of the sum over K (below)
  int shape = 0;
  {
    const bool planes3 = gsm == 2 && !v.mx && !v.symmetric;  // needs 256 rows of W per workgroup
    if (!planes3 && n128 * m32 <= 256) shape = 4;
    else if (!planes3 && n128 * m64 <= 256) shape = 2;
    else if (!planes3 && n128 * m128 <= 256) shape = 3;
    else if (n256 * m64 <= 256) shape = 1;
  }
  // The two smallest tiles run with two sets of waves, each on one half of K (their stages
  // are a serial chain; see the kernel): the sum over K is then (first half) + (second half).
  const int stages = v.K / 128;
  const int sets = (shape == 2 || shape == 4) && stages >= 8 ? 2 : 1;
  const int split_at = sets == 2 ? (stages + 1) / 2 : v.K;
  if (w_out) shape = 0;
  const long long tiles_n = (shape == 2 || shape == 3 || shape == 4) ? n128 : n256;
  const long long tiles_m = (shape == 0 || shape == 3) ? m128 : shape == 4 ? m32 : m64;
  if (M < 65 || n256 * m128 < 8 || tiles_n * tiles_m > 0x7FFFFFFFLL) return false;
  if ((long long)v.N * v.K / 2 >= (1LL << 32) || (long long)M * v.K * 2 >= (1LL << 32)) return false;
  // one FP16 scale per stage: the dword around it must lie inside the array
  if (gsm == 0 && (((long long)v.N * v.G) & 1)) return false;
  if ((((uintptr_t)v.q | (uintptr_t)x) & 15) || ((uintptr_t)v.scales & 3)) return false;
  if (!v.mx && !v.symmetric && (v.zeros == nullptr || ((uintptr_t)v.zeros & 3))) return false;
  if (w_out && ((uintptr_t)w_out & 15)) return false;
  // grids of more than one round: 256 x 256 tiles where they halve the rounds
  if (!w_out && try_tile256(v, x, c, M, s, 256, err)) return true;
  const int tn = (int)tiles_n, tm = (int)tiles_m;
  if (v.mx) *err = launch_hook<2, 2>(v, x, c, w_out, M, s, tn, tm, shape, sets, split_at);
  else if (v.symmetric) *err = launch_gsm<0>(gsm, v, x, c, w_out, M, s, tn, tm, shape, sets, split_at);
  else *err = launch_gsm<1>(gsm, v, x, c, w_out, M, s, tn, tm, shape, sets, split_at);
  return true;
}

}  // namespace w4k
