// Decode-batch W4A16 / MXFP4 GEMM (M <= 64) for long K (more than four 128-k chunks
// per wave: K = 4224 .. 16384 in whole chunks, the down-projection side of the usual
// MLP shapes).  mma.cuh:63-230 is the reference's kernel for this
// path.
//
// Same decomposition and the same order of additions as the resident-activation
// kernel of gemm_decode_resident.hip and the K-split kernel of gemm_mfma.hip (which
// serves the hooked calls): a workgroup owns one 16-row tile of W, its 8 waves split
// K by 128-k chunks (wave w owns chunks [CH w, CH (w + 1))), partial sums meet in LDS
// in wave order.  What differs is when things are asked for.  With K this long a
// 16-row tile is 90 .. 115 KB of codes and its MFMAs want 350 .. 460 KB of activations;
// N = 4096 gives one workgroup per compute unit, so nothing else runs on the unit
// while a workgroup waits.  The resident kernel requests everything, waits for all of
// it and then multiplies: the stream (5 .. 6 us) and the expansion of the codes
// (3 .. 4 us of vector-ALU work per SIMD) come one after the other.  Here a wave runs
// a software pipeline over its chunks:
//   * its LDS region is a ring of 2 to 4 units of x (a unit: one chunk of one tile of 16
//     activation rows); unit u + NBUF is requested (global_load_lds_dwordx4, whole
//     lines, XOR-swizzled) as soon as unit u has been read back into registers;
//   * codes are requested a unit (two chunks) at a time, two units ahead; with an even
//     number of chunks per wave and rows of whole 256-byte pairs of lines the two
//     loads of a unit take whole lines (rows 0..7, rows 8..15) and pair_fix()
//     restores the operand layout, as in the resident kernel;
//   * every wait is a vmcnt with the number of younger requests, known at compile
//     time from the fixed issue order (lk_schedule()).
// The memory path serves a compute unit's requests in order, so looking further
// ahead with the codes than with the activations gains nothing: what matters is that
// a wave multiplies chunk i while chunks i + 1 .. i + 4 are on their way.
#include <atomic>

#include <type_traits>
#include <utility>

#include "dq.cuh"
#include "kernels.h"

namespace w4k {
namespace {

// f(integral_constant<int, 0>), f(integral_constant<int, 1>), ...: a loop whose index is
// a constant expression inside the body (wait counts are instruction immediates)
template <class F, int... I>
__device__ __forceinline__ void lk_for(F&& f, std::integer_sequence<int, I...>) {
  (f(std::integral_constant<int, I>{}), ...);
}

typedef __attribute__((address_space(3))) void* lds_ptr;
constexpr int LK_WAVES = 8, LK_THREADS = 64 * LK_WAVES;
constexpr int LK_MAX_M = 64;
// A unit of activations is one 128-k chunk of one tile of 16 rows (NQ KB: NQ quads of
// rows).  Units in a wave's ring: with one row tile as many as 8 KB hold, at least 2 and
// at most 4 (deeper rings measured no better, and a workgroup that stays within 64 KB
// lets a compute unit hold two of them when N gives it more than one tile: N = 8192,
// K = 8192, M = 16: 18.6 -> 17.2 us); with several row tiles four units of 4 KB, so that
// the stream from L2 goes on while a unit is read back into registers (with whole
// chunks of 2 or 4 units as the granule the two took turns).  Units of codes (two
// chunks) requested ahead: half as many as chunks in the ring, at least 2.
constexpr int lk_nbuf(int MT, int NQ) {
  return MT > 1 ? 4 : 8 / NQ < 2 ? 2 : 8 / NQ < 4 ? 8 / NQ : 4;
}
constexpr int lk_lau(int MT, int NQ) { return lk_nbuf(MT, NQ) / MT / 2 > 2 ? lk_nbuf(MT, NQ) / MT / 2 : 2; }
constexpr int lk_waitcnt_vm(int n) { return (n & 0xF) | ((n >> 4) << 14) | 0x0F70; }
extern __shared__ __attribute__((aligned(16))) uint8_t lk_lds[];

__device__ __forceinline__ h8 lk_expand_word(uint32_t w, h2 cneg, h2 s2, uint32_t mask, uint32_t magic) {
  u4 out;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const uint32_t p = __builtin_amdgcn_perm(0u, w, 0x0c000c00u | (uint32_t)(i << 16) | (uint32_t)i);
    const uint32_t v = (p & mask) | magic;
    out[i] = as_u32((as_h2(v) + cneg) * s2);
  }
  return __builtin_bit_cast(h8, out);
}

// The issue order of a wave, replayed at compile time.  allowed[u]: how many vector
// memory requests may still be outstanding when unit u of the activations (chunk
// u / MT, row tile u % MT) is read back -- those issued after the last one it needs;
// the first unit of a chunk also needs the chunk's codes.  NSC: parameter loads per chunk.
template <int UN>
struct LkSched {
  int allowed[UN];
  int peak;
};
template <int CH, int MT, int NQ, int NSC>
constexpr LkSched<CH * MT> lk_schedule() {
  constexpr int NBUF = lk_nbuf(MT, NQ), LAU = lk_lau(MT, NQ), UN = CH * MT;
  LkSched<UN> s{};
  int xlast[UN] = {}, clast[CH] = {};
  int seq = NSC * CH;  // the parameter loads go first
  int cu = 0;          // units of codes issued
  auto codes = [&](int u) {
    if (2 * u >= CH) return;
    seq += (2 * u + 1 < CH) ? 2 : 1;
    clast[2 * u] = seq - 1;
    if (2 * u + 1 < CH) clast[2 * u + 1] = seq - 1;
  };
  for (int u = 0; u < NBUF && u < UN; ++u) {
    seq += NQ, xlast[u] = seq - 1;
    if ((u + 1) % (2 * MT) == 0 && cu < LAU) codes(cu++);
  }
  while (cu < LAU) codes(cu++);
  s.peak = seq;
  int done = -1;  // the youngest request known to have landed
  for (int u = 0; u < UN; ++u) {
    int need = xlast[u];
    if (clast[u / MT] > need) need = clast[u / MT];
    if (need > done) done = need;
    s.allowed[u] = seq - 1 - done;
    if (seq - 1 - done > s.peak) s.peak = seq - 1 - done;
    if (u + NBUF < UN) seq += NQ, xlast[u + NBUF] = seq - 1;
    if (u % MT == MT - 1 && (u / MT) % 2 == 0) codes(u / MT / 2 + LAU);
  }
  return s;
}

// FMT: 0 W4 symmetric, 1 W4 with zero-points, 2 MXFP4.  CH chunks of 128 k per wave
// (K any multiple of 128 with ceil(K / 128 / 8) == CH; chunks past the end of the row
// are fetched from a clamped address and meet zero activations).  gs_shift: log2(gs) if
// gs is a power of two, else -1.  MT tiles of 16 activation rows (grid.y walks M in
// steps of 16 MT).  G: groups (W4) or blocks (MXFP4) per row.
// NQ: quads of activation rows fetched per row tile (with one row tile, M <= 4 NQ: the
// quads past M would repeat row M - 1 and feed columns of the product that are never
// stored; they are left out and those columns are computed from whatever the buffer
// holds).  Arguments are scalars and pointers so that they arrive preloaded in SGPRs.
template <int FMT, int CH, int MT, int NQ>
__global__ __launch_bounds__(LK_THREADS) void mfma_decode_longk_kernel(
    const uint32_t* __restrict__ q, const void* __restrict__ scales,
    const uint32_t* __restrict__ zeros, const w4_half* __restrict__ x, w4_half* __restrict__ c,
    const int N, const int K, const int M, const int gs_shift, const int G, const int gs) {
  constexpr bool MX = FMT == 2;
  constexpr int NBUF = lk_nbuf(MT, NQ), LK_LAU = lk_lau(MT, NQ), NSC = FMT == 1 ? 2 : 1, UN = CH * MT;
  constexpr LkSched<UN> SCH = lk_schedule<CH, MT, NQ, NSC>();
  static_assert(SCH.peak < 64, "vmcnt is a 6-bit counter");
  static_assert(SCH.allowed[UN - 1] == 0, "the last unit waits for every request");
  static_assert(MT == 1 || NQ == 4, "several row tiles: whole tiles of 16 rows");
  constexpr int XBYTES = NBUF * NQ * 1024;  // the wave's ring: NBUF units of NQ KB
  const int WPR = K >> 3, nchunks = K >> 7;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r = lane & 15, b = lane >> 4;
  const int m0 = (int)blockIdx.y * (16 * MT);
  const int tile = (int)blockIdx.x;
  const size_t nrow = (size_t)(tile * 16 + r);
  auto chunk_of = [&](int i) { return min(wave * CH + i, nchunks - 1); };

  // ---- requests ----
  const uint32_t region = (uint32_t)(uintptr_t)(lds_ptr)lk_lds + (uint32_t)wave * XBYTES;
  const char* xb = (const char*)x;
  // unit u = (chunk u / MT, row tile u % MT) of this wave's slice of x -> buffer u % NBUF:
  // block rq = rows 4 rq .. + 3 of the tile; lane l fetches row l / 16 of the four,
  // 16-byte piece (l % 16) ^ (row % 16) of the chunk's 256 bytes.  Rows past M repeat
  // row M - 1.
  auto request_x = [&](int u) {
    const int cidx = chunk_of(u / MT), mt = u % MT;
#pragma unroll
    for (int rq = 0; rq < NQ; ++rq) {
      const int r16 = 4 * rq + (lane >> 4), row = m0 + 16 * mt + r16;
      const uint32_t off = (uint32_t)min(row, M - 1) * (uint32_t)(K * 2) + (uint32_t)cidx * 256u +
                           (uint32_t)(((lane & 15) ^ r16) * 16);
      const uint32_t dst = region + (uint32_t)((u % NBUF) * NQ + rq) * 1024u;
      asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1"
                   :
                   : "v"(off), "s"(xb), "s"(dst)
                   : "memory", "m0");
    }
  };
  constexpr bool PAIRC = CH % 2 == 0;
  const bool paired = PAIRC && (K & 255) == 0;
  u4 qw[CH];
  const uint32_t* qr = q + nrow * WPR;
  const uint32_t* qa = q + (nrow - (size_t)(r & 8)) * WPR;  // row r % 8 of the tile
  const uint32_t* qb = qa + (size_t)8 * WPR;                // row 8 + r % 8
  const int pa = 4 * (b + 4 * (r >> 3)), pb = 4 * (b + 4 * ((r >> 3) ^ 1));  // piece, in words
  // Code loads are inline assembly like the activation requests: the compiler then
  // places no waits of its own in the pipeline (it does not count the requests it
  // cannot see, so its waits for these registers would drain nearly everything in
  // flight), and the explicit waits below cover both.
  auto load16 = [&](u4& dst, const uint32_t* ptr) {
    asm volatile("global_load_dwordx4 %0, %1, off nt" : "=&v"(dst) : "v"(ptr) : "memory");
  };
  auto request_codes = [&](int u) {
    const int i = 2 * u;
    if (PAIRC && paired) {
      const int w0 = 16 * min(wave * CH + i, nchunks - 2);  // nchunks is even here
      load16(qw[i], qa + w0 + pa);
      load16(qw[i + 1], qb + w0 + pb);
    } else {
      load16(qw[i], qr + chunk_of(i) * 16 + 4 * b);
      if (i + 1 < CH) load16(qw[i + 1], qr + chunk_of(i + 1) * 16 + 4 * b);
    }
  };
  auto pair_fix = [&](int u) {
    if (!(PAIRC && paired)) return;
    const int i = 2 * u;
    const bool lo = r < 8;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const uint32_t a = qw[i][e], bb = qw[i + 1][e];
      qw[i][e] = lo ? a : bb;
      // row_ror:8 -- lane r of each row of 16 takes the value of lane r ^ 8
      qw[i + 1][e] = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)(lo ? bb : a), 0x128, 0xF, 0xF, true);
    }
  };

  // group parameters of this lane's slice of every chunk, first: they are small and
  // every later wait then covers them
  uint32_t sc[CH], zw[CH];
  int gidx[CH];
#pragma unroll
  for (int i = 0; i < CH; ++i) {
    const int k = chunk_of(i) * 128 + 32 * b;
    gidx[i] = MX ? (k >> 5) : gs_shift >= 0 ? (k >> gs_shift) : k / gs;
    if (MX) {
      const uint8_t* sp = (const uint8_t*)scales + nrow * G + gidx[i];
      asm volatile("global_load_ubyte %0, %1, off" : "=&v"(sc[i]) : "v"(sp) : "memory");
    } else {
      const uint16_t* sp = (const uint16_t*)scales + nrow * G + gidx[i];
      asm volatile("global_load_ushort %0, %1, off" : "=&v"(sc[i]) : "v"(sp) : "memory");
      if (FMT == 1) {
        const uint32_t* zp = zeros + nrow * words(G) + (gidx[i] >> 3);
        asm volatile("global_load_dword %0, %1, off" : "=&v"(zw[i]) : "v"(zp) : "memory");
      }
    }
  }
  __builtin_amdgcn_sched_barrier(0);
  // (the scheduling barriers pin the order that lk_schedule() replays)
  {
    int cu = 0;
#pragma unroll
    for (int u = 0; u < NBUF && u < UN; ++u) {
      request_x(u);
      __builtin_amdgcn_sched_barrier(0);
      if ((u + 1) % (2 * MT) == 0 && cu < LK_LAU) {
        if (2 * cu < CH) request_codes(cu);
        ++cu;
        __builtin_amdgcn_sched_barrier(0);
      }
    }
#pragma unroll
    for (int k = 0; k < LK_LAU; ++k)
      if (k >= cu && 2 * k < CH) request_codes(k);
    __builtin_amdgcn_sched_barrier(0);
  }
  uint32_t mask = 0x00F0000Fu, magic = 0x54006400u;
  asm volatile("" : "+s"(mask));   // opaque: as literals they cost two instructions
  asm volatile("" : "+v"(magic));  // instead of one and-or
  f4 acc[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) acc[mt] = f4{0.f, 0.f, 0.f, 0.f};

  const uint8_t* mine = lk_lds + wave * XBYTES;
  u4 xv[MT][4];  // B operands: MFMA j contracts k = 128 chunk + 32 b + 8 j .. + 7 = piece 4 b + j
  lk_for([&](auto uc) {
    constexpr int u = decltype(uc)::value, i = u / MT, mt = u % MT;
    __builtin_amdgcn_s_waitcnt(lk_waitcnt_vm(SCH.allowed[u]));
    if (mt == 0) {
      // the registers of this chunk's codes are defined from here on
      asm volatile("" : "+v"(qw[i]), "+v"(sc[i]));
      if (FMT == 1) asm volatile("" : "+v"(zw[i]));
      if (i % 2 == 0 && i + 1 < CH) asm volatile("" : "+v"(qw[i + 1]));
    }
    __builtin_amdgcn_sched_barrier(0);
    if (mt == 0 && i % 2 == 0 && i + 1 < CH) pair_fix(i / 2);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      // (lanes of rows past the fetched quads read the last fetched one)
      xv[mt][j] = *(const u4*)(mine + ((u % NBUF) * NQ + min(r >> 2, NQ - 1)) * 1024 +
                               ((r & 3) * 16 + ((4 * b + j) ^ r)) * 16);
    }
    if (wave * CH + i >= nchunks) {  // a chunk past the end of the row: zero activations
#pragma unroll
      for (int j = 0; j < 4; ++j) xv[mt][j] = u4{0u, 0u, 0u, 0u};
      // keeps this a branch that only the ragged tail takes (as selects it is 16
      // instructions per chunk for every wave, a fifth of the chunk's vector-ALU work)
      asm volatile("" ::: "memory");
    }
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): the buffer is free
    __builtin_amdgcn_sched_barrier(0);
    if (u + NBUF < UN) request_x(u + NBUF);
    __builtin_amdgcn_sched_barrier(0);
    if (mt != MT - 1) return;  // the chunk's other row tiles first
    if (i % 2 == 0 && 2 * (i / 2 + LK_LAU) < CH) request_codes(i / 2 + LK_LAU);
    __builtin_amdgcn_sched_barrier(0);

    h2 cneg, s2;
    float sf = 0.f;
    if (MX) {
      sf = mx_scale(sc[i]);
    } else {
      const uint32_t z = FMT == 1 ? ((zw[i] >> (4 * (gidx[i] & 7))) & 0xFu) : 8u;
      cneg = as_h2(0xD400E400u | (z << 20) | z);
      s2 = splat_bits(sc[i]);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      h8 a;
      if (MX) {
        h2 n4[4];
        dq_mx(qw[i][j], sf, n4);
        a = __builtin_bit_cast(h8, u4{as_u32(n4[0]), as_u32(n4[1]), as_u32(n4[2]), as_u32(n4[3])});
      } else {
        a = lk_expand_word(qw[i][j], cneg, s2, mask, magic);
      }
#pragma unroll
      for (int m2 = 0; m2 < MT; ++m2)
        acc[m2] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, __builtin_bit_cast(h8, xv[m2][j]), acc[m2],
                                                         0, 0, 0);
    }
  }, std::make_integer_sequence<int, UN>{});

  // Fixed-order combine of the 8 K slices: entry mt of wave w goes to red[w][mt]; wave
  // e < MT then sums entry e in wave order and stores it.  The rings are free once
  // every wave is here.
  __syncthreads();
  f4* red = (f4*)lk_lds;  // [LK_WAVES][MT][64]
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) red[(wave * MT + mt) * 64 + lane] = acc[mt];
  __syncthreads();
  if (wave < MT) {
    const int mt = wave;
    f4 s = red[mt * 64 + lane];
#pragma unroll
    for (int w = 1; w < LK_WAVES; ++w) s += red[(w * MT + mt) * 64 + lane];
    const int m = m0 + 16 * mt + r;
    if (m < M) {  // lane: activation row m, weight rows 16 tile + 4 b .. + 3
      uint16_t hv[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const _Float16 hh = (_Float16)s[k];
        hv[k] = __builtin_bit_cast(uint16_t, hh);
      }
      *(u2*)(c + (size_t)m * N + tile * 16 + 4 * b) =
          u2{hv[0] | ((uint32_t)hv[1] << 16), hv[2] | ((uint32_t)hv[3] << 16)};
    }
  }
}

// Chunks per wave if K is this kernel's (whole chunks, 2 .. 16 per wave: 1152 .. 16384), else 0.
int longk_chunks(int K) {
  if (K % 128) return 0;
  const int per_wave = (K / 128 + LK_WAVES - 1) / LK_WAVES;
  return (per_wave >= 2 && per_wave <= 16) ? per_wave : 0;
}

// Compute units of the current device (per-device cache); 0 on error.
int lk_cus() {
  static std::atomic<int> cached[64] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 0;
  if (dev >= 0 && dev < 64 && cached[dev]) return cached[dev];
  int n = 0;
  if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
  if (dev >= 0 && dev < 64) cached[dev] = n;
  return n;
}

template <int FMT, int CH, int MT, int NQ>
hipError_t longk_go(const WView& v, const w4_half* x, w4_half* c, int M, hipStream_t s) {
  constexpr int lds_bytes = LK_WAVES * lk_nbuf(MT, NQ) * NQ * 1024;
  static std::atomic<bool> granted[64] = {};  // more than 64 KB of LDS has to be granted per device, once
  int dev = 0;
  if (hipError_t e = hipGetDevice(&dev); e != hipSuccess) return e;
  if (lds_bytes > 65536 && (dev < 0 || dev >= 64 || !granted[dev])) {
    const hipError_t e = hipFuncSetAttribute((const void*)mfma_decode_longk_kernel<FMT, CH, MT, NQ>,
                                             hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
    if (e != hipSuccess) return e;
    if (dev >= 0 && dev < 64) granted[dev] = true;
  }
  const bool pow2 = !v.mx && (v.gs & (v.gs - 1)) == 0;
  const dim3 grid((unsigned)(v.N / 16), (unsigned)((M + 16 * MT - 1) / (16 * MT)));
  mfma_decode_longk_kernel<FMT, CH, MT, NQ><<<grid, LK_THREADS, lds_bytes, s>>>(
      v.q, v.scales, v.zeros, x, c, v.N, v.K, M, pow2 ? __builtin_ctz((unsigned)v.gs) : -1,
      v.mx ? v.B : v.G, v.gs);
  return hipGetLastError();
}

template <int FMT, int CH>
hipError_t longk_m(const WView& v, const w4_half* x, w4_half* c, int M, hipStream_t s) {
  if (M <= 4) return longk_go<FMT, CH, 1, 1>(v, x, c, M, s);
  if (M <= 8) return longk_go<FMT, CH, 1, 2>(v, x, c, M, s);
  if (M <= 12) return longk_go<FMT, CH, 1, 3>(v, x, c, M, s);
  if (M <= 16) return longk_go<FMT, CH, 1, 4>(v, x, c, M, s);
  if (M <= 32) return longk_go<FMT, CH, 2, 4>(v, x, c, M, s);
  return longk_go<FMT, CH, 4, 4>(v, x, c, M, s);  // grid.y walks 64 rows at a time
}

template <int FMT>
hipError_t longk_fmt(const WView& v, const w4_half* x, w4_half* c, int M, hipStream_t s) {
  switch (longk_chunks(v.K)) {
    case 2: return longk_m<FMT, 2>(v, x, c, M, s);
    case 3: return longk_m<FMT, 3>(v, x, c, M, s);
    case 4: return longk_m<FMT, 4>(v, x, c, M, s);
    case 5: return longk_m<FMT, 5>(v, x, c, M, s);
    case 6: return longk_m<FMT, 6>(v, x, c, M, s);
    case 7: return longk_m<FMT, 7>(v, x, c, M, s);
    case 8: return longk_m<FMT, 8>(v, x, c, M, s);
    case 9: return longk_m<FMT, 9>(v, x, c, M, s);
    case 10: return longk_m<FMT, 10>(v, x, c, M, s);
    case 11: return longk_m<FMT, 11>(v, x, c, M, s);
    case 12: return longk_m<FMT, 12>(v, x, c, M, s);
    case 13: return longk_m<FMT, 13>(v, x, c, M, s);
    case 14: return longk_m<FMT, 14>(v, x, c, M, s);
    case 15: return longk_m<FMT, 15>(v, x, c, M, s);
    case 16: return longk_m<FMT, 16>(v, x, c, M, s);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace

// 5 to 16 whole chunks of 128 k per wave (2 to 4 on thin grids, see below), whole 16-row
// tiles, a lane's 32-k slice inside one group, M <= 64, 16-byte aligned codes and
// activations.
bool decode_longk_applies(const WView& v, const w4_half* x, const w4_half* c, int M) {
  if (M < 1 || M > LK_MAX_M || v.N % 16 || longk_chunks(v.K) == 0) return false;
  if (!v.mx && v.gs % 32) return false;
  if ((((uintptr_t)v.q | (uintptr_t)x) & 15) || ((uintptr_t)c & 7)) return false;
  // more tiles than compute units and more than 12 to 16 activation rows: the kernel that shares a
  // workgroup's activations between two tiles is ahead where it exists (8, 11, 14 chunks per wave)
  if (decode_resident_shares_long_k(v, x, c, M)) return false;
  // K up to 5120 on grids of more than one tile per compute unit, W4: from M = 9 the kernel
  // that shares a workgroup's activations between several tiles is ahead (N = 16384,
  // K = 5120, M = 16 / 32 / 64: 17.7 / 20.0 / 35.8 us against 21.3 / 31.3 / 42.0; M = 8: 17.2 against 17.0)
  if (longk_chunks(v.K) == 5 && !v.mx && M > 8 && v.N / 16 > lk_cus()) return false;
  if (longk_chunks(v.K) < 5) {
    // Shorter K: only where the kernels that share x between the tiles of a workgroup
    // would have one tile per workgroup too (N / 16 <= compute units).  At K = 2048 and
    // 4096, the resident kernel's own, this one is ahead while few quads of x are
    // fetched and most compute units have a tile (N = 4096, K = 4096, M = 5 / 8: 5.5 ->
    // 4.8 / 5.0 us; M = 16: 5.6 -> 5.9; N = 2048, M = 8: 5.35 -> 5.66).
    const int tiles = v.N / 16, cus = lk_cus();
    if (cus < 1 || tiles > cus) return false;
    if ((v.K == 2048 || v.K == 4096) && (M > 8 || 2 * tiles <= cus)) return false;
  }
  return true;
}

// Precondition: decode_longk_applies(v, x, c, M); no hook.
hipError_t launch_decode_longk(const WView& v, const w4_half* x, w4_half* c, int M, hipStream_t s) {
  if (!decode_longk_applies(v, x, c, M)) return hipErrorInvalidValue;
  if (v.mx) return longk_fmt<2>(v, x, c, M, s);
  return v.symmetric ? longk_fmt<0>(v, x, c, M, s) : longk_fmt<1>(v, x, c, M, s);
}

}  // namespace w4k
