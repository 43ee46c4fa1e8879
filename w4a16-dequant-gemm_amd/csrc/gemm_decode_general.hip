// Decode-batch W4A16 GEMM (M <= 64) for the shapes the resident-activation kernel of
// gemm_decode_resident.hip does not take: group sizes that are no multiple of 32 (a
// lane's 32-k slice then spans several groups) and K that is no multiple of 128
// (K % 8 == 0: whole packed words; rows of words are then only 4-byte aligned).
// mma.cuh:63-230 is the reference's kernel for this path: any gs % 8 == 0, any K,
// zero-padded edges.
//
// Same structure as the resident-activation kernel -- 8 waves split K by 128-k
// chunks, a workgroup takes T 16-row tiles and brings its activations in once
// (global_load_lds_dwordx4 into each wave's own LDS region, XOR-swizzled), partial
// sums meet in LDS in wave order -- and the same order of additions as
// mfma_decode_kernel, which serves the hooked calls of these shapes.  What differs:
//  * group parameters come through LDS.  The scales of a tile's 16 rows are one
//    contiguous 32-byte-aligned run of 32 G bytes (the zero-point words one of
//    64 words(G) bytes): the workgroup copies the runs of its T tiles with 16-byte
//    loads, and every lane then reads the scale and the zero-point word of each of
//    its packed words from LDS (group indices computed once per kernel; a lookup per
//    word, or two per slice where gs >= 32 allows it).
//    Gathering them from memory costs a separate request per (row, group) touched:
//    at gs = 48, N = 11008 that was as much as the shared activations saved.
//  * rows of packed words are read with 16-byte loads at 4-byte aligned addresses
//    (the memory path takes them at 0.95 of the aligned rate); a slice that runs past
//    the end of its row is read word by word with the index clamped to the row.
//  * the last chunk of a row may be partial: its activations beyond K are fetched
//    from a clamped address and zeroed on the way to the MFMA operands.
#include <atomic>

#include "dq.cuh"
#include "kernels.h"

namespace w4k {
namespace {

typedef __attribute__((address_space(3))) void* lds_ptr;
constexpr int DG_WAVES = 8, DG_THREADS = 64 * DG_WAVES;
constexpr int dg_waitcnt_vm(int n) { return (n & 0xF) | ((n >> 4) << 14) | 0x0F70; }
extern __shared__ __attribute__((aligned(16))) uint8_t dg_lds[];

// Eight codes of a packed word -> eight FP16 weights in k order (as in the
// resident-activation kernel): cneg = packed {-(1024 + z), -(64 + z)}, s2 = the scale
// in both halves, mask / magic = 0x00F0000F / 0x54006400 held in registers.
__device__ __forceinline__ h8 dg_expand_word(uint32_t w, h2 cneg, h2 s2, uint32_t mask, uint32_t magic) {
  u4 out;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const uint32_t p = __builtin_amdgcn_perm(0u, w, 0x0c000c00u | (uint32_t)(i << 16) | (uint32_t)i);
    const uint32_t v = (p & mask) | magic;
    out[i] = as_u32((as_h2(v) + cneg) * s2);
  }
  return __builtin_bit_cast(h8, out);
}

// ASYM: zero-points.  CH = ceil(ceil(K / 128) / 8) chunks per wave.  T tiles of 16 rows
// per workgroup (tile blockIdx.x + gridDim.x t), MT tiles of 16 activation rows
// (blockIdx.y walks M in steps of 16 MT); CPX, if not 0, chunks of x per phase.  GM: how a
// slice's groups are looked up (2: gs >= 32, first and last word only; 1: gs = 8 or 16,
// one zero-point word per slice; 0: per word).  A tile's scales are copied with PS = 3 16-byte
// loads per thread (2 G <= 1536 of them; indices past the run repeat its last piece and
// are not written).  Arguments are scalars and pointers so that they arrive preloaded
// in SGPRs.
template <bool ASYM, int CH, int T, int MT, int CPX, int GM>
__global__ __launch_bounds__(DG_THREADS) void mfma_decode_general_kernel(
    const uint32_t* __restrict__ q, const w4_half* __restrict__ scales,
    const uint32_t* __restrict__ zeros, const w4_half* __restrict__ x, w4_half* __restrict__ c,
    const int N, const int K, const int gs, const int gs_shift, const int G, const int M,
    const int tiles) {
  constexpr int PS = 3;
  const int WPR = K >> 3, nchunks = (K + 127) >> 7, WG = (G + 7) >> 3;
  // chunks per phase: as many as 16 KB per wave hold (4 / MT), or CPX if given (fewer
  // chunks per phase leave LDS for the parameter blocks of more tiles)
  constexpr int CPD = CPX > 0 ? CPX : 4 / MT;
  constexpr int CP = CPD < CH ? CPD : CH;
  constexpr int PH = (CH + CP - 1) / CP;              // phases (the last may be partial)
  constexpr int XBYTES = MT * CP * 4096;              // the wave's LDS region
  const int SB = 32 * G, ZB = ASYM ? 64 * WG : 0;     // a tile's scale / zero-point bytes
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r = lane & 15, b = lane >> 4;
  const int m0 = (int)blockIdx.y * (16 * MT);
  // chunk i of this wave (clamped to the row's last chunk) and this lane's first k in it
  auto chunk_of = [&](int i) { return min(wave * CH + i, nchunks - 1); };
  auto lane_k = [&](int i) { return chunk_of(i) * 128 + 32 * b; };

  int tile_of[T];
#pragma unroll
  for (int t = 0; t < T; ++t) tile_of[t] = min((int)blockIdx.x + (int)gridDim.x * t, tiles - 1);

  // ---- requests: activations of phase 0, codes of tile 0, group parameters, other codes ----
  const uint32_t region = (uint32_t)(uintptr_t)(lds_ptr)dg_lds + (uint32_t)wave * XBYTES;
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
          const int cidx = chunk_of(ph * CP + cc);
          // 16-byte piece (lane % 16) ^ r16 of the chunk's 256 bytes; pieces past K repeat piece 0
          int piece = (lane & 15) ^ r16;
          if (cidx * 128 + piece * 8 >= K) piece = 0;
          const uint32_t off = (uint32_t)min(row, M - 1) * (uint32_t)(K * 2) + (uint32_t)cidx * 256u +
                               (uint32_t)(piece * 16);
          const uint32_t dst = region + (uint32_t)((mt * CP + cc) * 4 + rq) * 1024u;
          asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1"
                       :
                       : "v"(off), "s"(xb), "s"(dst)
                       : "memory", "m0");
        }
  };
  // With an even number of chunks per wave and rows that are whole 128-byte lines the
  // two loads of chunks 2P, 2P + 1 take whole lines (rows 0..7 of the tile in the
  // first, 8..15 in the second; lane (r, b) fetches piece b + 4 (r / 8) resp.
  // b + 4 (1 - r / 8) of its line) and pair_fix() restores the operand layout with a
  // select and a rotation of the rows of 16 lanes by 8, as in the resident-activation
  // kernel: loads of 64 bytes out of every line run at 0.8 of the rate.
  const bool paired = CH % 2 == 0 && (K & 255) == 0;
  u4 qw[T][CH];
  auto load_tile = [&](int t) {
    if (paired) {
      const uint32_t* qa = q + (size_t)(tile_of[t] * 16 + (r & 7)) * WPR;
      const uint32_t* qb = qa + (size_t)8 * WPR;
      const int pa = 4 * (b + 4 * (r >> 3)), pb = 4 * (b + 4 * ((r >> 3) ^ 1));
#pragma unroll
      for (int i = 0; i + 1 < CH; i += 2) {
        const int w0 = 16 * min(wave * CH + i, nchunks - 2);  // nchunks is even here
        qw[t][i] = __builtin_nontemporal_load((const u4*)(qa + w0 + pa));
        qw[t][i + 1] = __builtin_nontemporal_load((const u4*)(qb + w0 + pb));
      }
      return;
    }
    const uint32_t* qr = q + (size_t)(tile_of[t] * 16 + r) * WPR;
#pragma unroll
    for (int i = 0; i < CH; ++i) {
      const int w0 = lane_k(i) >> 3;
      if (w0 + 4 <= WPR) {
        qw[t][i] = __builtin_nontemporal_load((const u4*)(qr + w0));
      } else {  // the slice runs past the row: word by word, clamped (those words meet zero activations)
#pragma unroll
        for (int j = 0; j < 4; ++j) qw[t][i][j] = __builtin_nontemporal_load(qr + min(w0 + j, WPR - 1));
      }
    }
  };
  auto pair_fix = [&](int t) {
    if (!paired) return;
    const bool lo = r < 8;
#pragma unroll
    for (int i = 0; i + 1 < CH; i += 2)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const uint32_t a = qw[t][i][e], bb = qw[t][i + 1][e];
        qw[t][i][e] = lo ? a : bb;
        qw[t][i + 1][e] = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)(lo ? bb : a), 0x128, 0xF, 0xF, true);
      }
  };
  request_x(0);
  load_tile(0);
  u4 sv[T][PS], zv[T];
#pragma unroll
  for (int t = 0; t < T; ++t) {
    const u4* sp = (const u4*)((const uint8_t*)scales + (size_t)tile_of[t] * SB);
#pragma unroll
    for (int ps = 0; ps < PS; ++ps) {
      const int i = min(ps * DG_THREADS + (int)threadIdx.x, SB / 16 - 1);
      sv[t][ps] = sp[i];
    }
    if (ASYM) {
      const u4* zp = (const u4*)((const uint8_t*)zeros + (size_t)tile_of[t] * ZB);
      zv[t] = zp[min((int)threadIdx.x, ZB / 16 - 1)];
    }
  }
  // the codes of tile t + 1 are requested just before tile t is multiplied (see the
  // resident-activation kernel: a wave that has to place every tile's loads first
  // starts its arithmetic late)
  if (T > 1) load_tile(1);
  __builtin_amdgcn_sched_barrier(0);  // every request above is issued before the wait below

  // Group of each packed word of this lane (the same for every tile), as byte offsets
  // into a tile's parameter block: scale at 2 (r G + g), zero-point word at
  // SB + 4 (r WG + g / 8), nibble g % 8.
  // G2 (gs >= 32): the four words of a lane's 32-k slice lie in at most two groups, that
  // of the first word and that of the last; only those two are looked up, and the
  // words between take one or the other (four LDS reads and ten vector instructions
  // less per slice: 13.2 -> 12.4 us at gs = 48, M = 8).
  // GM == 1 (gs = 8 or 16, which divide 32): the groups of a slice start at a multiple of
  // 32 / gs, so their zero-points sit in one word, read once per slice.
  constexpr bool G2 = GM == 2, ZS = GM == 1;
  constexpr int NL = G2 ? 2 : 4;
  uint32_t soff[CH][NL], zoff[CH][NL], zsh[CH][NL];
  bool first[CH][2];  // G2: words 1 and 2 are in the first word's group
#pragma unroll
  for (int i = 0; i < CH; ++i) {
    int g4[4];
    groups_of_slice(lane_k(i), gs, gs_shift, G - 1, g4);
    first[i][0] = g4[1] == g4[0];
    first[i][1] = g4[2] == g4[0];
#pragma unroll
    for (int l = 0; l < NL; ++l) {
      const int g = g4[G2 ? 3 * l : l];
      soff[i][l] = (uint32_t)(r * G + g) * 2u;
      zoff[i][l] = (uint32_t)SB + (uint32_t)(r * WG + (g >> 3)) * 4u;
      zsh[i][l] = 4u * (uint32_t)(g & 7);
    }
  }

  // At most the codes of tile 1 may still be outstanding (CH vector loads; a wave that
  // issued word-by-word loads instead waits for more than it must): phase 0 of x, the
  // codes of tile 0 and the parameter loads have landed.
  __builtin_amdgcn_s_waitcnt(dg_waitcnt_vm(T > 1 ? CH : 0));
  const int PB = SB + ZB;  // parameter block of one tile, behind the x regions
  uint8_t* params = dg_lds + DG_WAVES * XBYTES;
#pragma unroll
  for (int t = 0; t < T; ++t) {
#pragma unroll
    for (int ps = 0; ps < PS; ++ps) {
      const int i = ps * DG_THREADS + (int)threadIdx.x;
      if (i < SB / 16) *(u4*)(params + t * PB + i * 16) = sv[t][ps];
    }
    if (ASYM && (int)threadIdx.x < ZB / 16) *(u4*)(params + t * PB + SB + threadIdx.x * 16) = zv[t];
  }
  __syncthreads();

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
    if (ph > 0) __builtin_amdgcn_s_waitcnt(dg_waitcnt_vm(0));  // later phases are the youngest requests
    // B operands: MFMA j of chunk i contracts k = lane_k(i) + 8 j .. + 7 = piece 4 b + j
    u4 xv[MT][CP][4];
    {
      const uint8_t* mine = dg_lds + wave * XBYTES;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int cc = 0; cc < CP; ++cc)
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const int i = ph * CP + cc;
            if (i >= CH) continue;
            xv[mt][cc][j] = *(const u4*)(mine + ((mt * CP + cc) * 4 + (r >> 2)) * 1024 +
                                         ((r & 3) * 16 + ((4 * b + j) ^ r)) * 16);
          }
    }
    // chunks past the row's last one, and k past K inside it, contribute nothing: a branch
    // that only the waves at the ragged end of the row take (as selects it was 16
    // vector instructions per chunk for every wave: 0.5 - 1.7 us per call)
#pragma unroll
    for (int cc = 0; cc < CP; ++cc) {
      const int i = ph * CP + cc;
      if (i >= CH) continue;
      if (wave * CH + i >= nchunks - ((K & 127) ? 1 : 0)) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
          for (int j = 0; j < 4; ++j)
            if (wave * CH + i >= nchunks || lane_k(i) + 8 * j >= K) xv[mt][cc][j] = u4{0u, 0u, 0u, 0u};
        asm volatile("" ::: "memory");
      }
    }
    if (ph + 1 < PH) {
      // the region is free once these reads have returned: ask for the next phase now
      __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
      __builtin_amdgcn_sched_barrier(0);
      request_x(ph + 1);
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
        if (t == 1) __builtin_amdgcn_s_waitcnt(dg_waitcnt_vm(NX1 + (T > 2 ? CH : 0)));
        else if (t + 1 < T) __builtin_amdgcn_s_waitcnt(dg_waitcnt_vm(CH));
        else __builtin_amdgcn_s_waitcnt(dg_waitcnt_vm(0));
      }
#pragma unroll
      for (int cc = 0; cc < CP; ++cc) {
        const int i = ph * CP + cc;
        if (i >= CH) continue;
        if (ph == 0 && cc == 0) pair_fix(t);
        const uint8_t* pt = params + t * PB;
        h2 cn[NL], sp[NL];
        uint32_t zword = 0u;
        if (ASYM && ZS) zword = *(const uint32_t*)(pt + zoff[i][0]);
#pragma unroll
        for (int l = 0; l < NL; ++l) {
          const uint32_t sbits = *(const uint16_t*)(pt + soff[i][l]);
          uint32_t z = 8u;
          if (ASYM) z = ((ZS ? zword : *(const uint32_t*)(pt + zoff[i][l])) >> zsh[i][l]) & 0xFu;
          cn[l] = as_h2(0xD400E400u | (z << 20) | z);
          sp[l] = splat_bits(sbits);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          h2 cneg, s2;
          if (!G2) {
            cneg = cn[j < NL ? j : 0], s2 = sp[j < NL ? j : 0];
          } else if (j == 0 || j == 3) {
            cneg = cn[j ? 1 : 0], s2 = sp[j ? 1 : 0];
          } else {
            cneg = first[i][j - 1] ? cn[0] : cn[1];
            s2 = first[i][j - 1] ? sp[0] : sp[1];
          }
          const h8 a = dg_expand_word(qw[t][i][j], cneg, s2, mask, magic);
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
            acc[t][mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, __builtin_bit_cast(h8, xv[mt][cc][j]),
                                                                acc[t][mt], 0, 0, 0);
        }
      }
    }
  }

  // Fixed-order combine of the 8 K slices (the x regions are free once every wave is
  // here): entry (t, mt) of wave w goes to red[w][t MT + mt]; wave w sums the entries
  // e = w, w + 8, ... in wave order and stores them.
  constexpr int E = T * MT;
  static_assert(DG_WAVES * E * 1024 <= DG_WAVES * XBYTES, "reduction buffer fits the x regions");
  __syncthreads();
  f4* red = (f4*)dg_lds;  // [DG_WAVES][E][64]
#pragma unroll
  for (int t = 0; t < T; ++t)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) red[(wave * E + t * MT + mt) * 64 + lane] = acc[t][mt];
  __syncthreads();
  for (int e = wave; e < E; e += DG_WAVES) {
    const int t = e / MT, mt = e % MT;
    const int tile = (int)blockIdx.x + (int)gridDim.x * t;
    if (tile >= tiles) continue;
    f4 s = red[e * 64 + lane];
#pragma unroll
    for (int w = 1; w < DG_WAVES; ++w) s += red[(w * E + e) * 64 + lane];
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

struct GeneralPlan {
  int ch, t, mt, cpx, lds;
};

// Most tiles per workgroup that an instantiation holds in registers without spilling
// (checked against the compiler's register counts).
constexpr int dg_tile_cap(int ch, int mt) { return (mt == 4 && ch == 5) ? 3 : 4; }
// What general_plan() can return: everything else is never compiled.
constexpr bool dg_planned(int ch, int t, int mt, int cpx) {
  if (t > dg_tile_cap(ch, mt)) return false;
  if (cpx == 2) return mt == 1 && ch > 2;
  if (cpx == 1) return mt == 2;
  return cpx == 0;
}

// LDS the device grants a workgroup (per-device cache); 0 on error.
int max_lds_bytes() {
  static std::atomic<int> cached[64] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 0;
  if (dev >= 0 && dev < 64) {
    if (const int have = cached[dev].load(std::memory_order_relaxed)) return have;
  }
  int n = 0;
  if (hipDeviceGetAttribute(&n, hipDeviceAttributeMaxSharedMemoryPerBlock, dev) != hipSuccess) return 0;
  if (dev >= 0 && dev < 64) cached[dev].store(n, std::memory_order_relaxed);
  return n;
}

int cu_count() {
  static std::atomic<int> cached[64] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 0;
  if (dev >= 0 && dev < 64) {
    if (const int have = cached[dev].load(std::memory_order_relaxed)) return have;
  }
  int n = 0;
  if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
  if (dev >= 0 && dev < 64) cached[dev].store(n, std::memory_order_relaxed);
  return n;
}

// Whether, and how, the kernel takes these arguments: W4 only, whole 16-row tiles,
// whole packed words, 1024 < K <= 5120 (two to five chunks per wave), M <= 64, aligned
// activations / outputs / parameter arrays, and LDS for the activations of a
// workgroup plus the parameter blocks of at least one tile.
bool general_plan(const WView& v, const w4_half* x, const w4_half* c, int M, GeneralPlan* out) {
  if (v.mx || M < 1 || M > 64 || v.N % 16 || v.K % 8 || v.gs % 8 || v.gs < 8) return false;
  const int nchunks = (v.K + 127) / 128, ch = (nchunks + DG_WAVES - 1) / DG_WAVES;
  if (ch < 2 || ch > 5) return false;
  if (((uintptr_t)x & 15) || ((uintptr_t)c & 7) || ((uintptr_t)v.q & 3)) return false;
  if (((uintptr_t)v.scales & 15) || (!v.symmetric && ((uintptr_t)v.zeros & 15))) return false;
  const int mt = M <= 16 ? 1 : M <= 32 ? 2 : 4;
  const int pb = 32 * v.G + (v.symmetric ? 0 : 64 * ((v.G + 7) / 8));
  const int ps = (2 * v.G + DG_THREADS - 1) / DG_THREADS;
  if (ps > 3 || (!v.symmetric && 4 * ((v.G + 7) / 8) > DG_THREADS)) return false;
  const int lds_max = max_lds_bytes(), cus = cu_count();
  if (lds_max < 1 || cus < 1) return false;
  // tiles per workgroup: enough that one workgroup per compute unit covers N, at most
  // four; with one activation row tile the x regions may shrink to two chunks per
  // phase to make room for the parameter blocks
  int want = (v.N / 16 + cus - 1) / cus;
  if (want > dg_tile_cap(ch, mt)) want = dg_tile_cap(ch, mt);
  auto fit = [&](int cpd, int* lds) {
    const int cp = cpd < ch ? cpd : ch;
    const int xbytes = DG_WAVES * mt * cp * 4096;
    int t = want;
    while (t > 0 && xbytes + t * pb > lds_max) --t;
    *lds = xbytes + t * pb;
    return t;
  };
  int lds = 0, cpx = 0;
  int t = fit(4 / mt, &lds);
  if (mt == 1 && ch > 2) {
    // Two chunks per phase: room for the parameter blocks of more tiles, and with as
    // many tiles the first activations are complete after half the requests, so the
    // waves start on tile 0 sooner (N = 11008, gs = 48, M = 8: 12.5 -> 11.8 us).
    int lds2 = 0;
    const int t2 = fit(2, &lds2);
    if (t2 >= t) t = t2, lds = lds2, cpx = 2;
  }
  if (mt == 2 && t < want) {
    // Large parameter blocks (gs = 8 at K = 4104: 20.6 KB per tile) leave room for fewer
    // tiles than the grid wants once the activations of 32 rows hold 128 KB.  With one
    // chunk per phase they hold 64 KB and a workgroup shares them between `want` tiles
    // again: N = 11008, K = 4104 / 4096, gs = 8, M = 32: 31.4 / 25.4 -> 20.9 / 16.2 us.
    // (64 rows as two such passes in grid.y measured no gain: 344 workgroups of 146 KB
    // are two rounds, 39.9 against 38.7 us.)
    int lds1 = 0;
    const int t1 = fit(1, &lds1);
    if (t1 > t) t = t1, lds = lds1, cpx = 1;
  }
  if (t < 1) return false;
  *out = GeneralPlan{ch, t, mt, cpx, lds};
  return true;
}

template <bool ASYM, int CH, int T, int MT, int CPX, int GM>
hipError_t general_gm(const WView& v, const w4_half* x, w4_half* c, int M, hipStream_t s,
                      const GeneralPlan& pl) {
  if constexpr (!dg_planned(CH, T, MT, CPX)) {
    return hipErrorInvalidValue;  // general_plan() never asks for it
  } else {
    // more than 64 KB of LDS has to be granted per device, once per instantiation
    static std::atomic<int> granted_bytes[64] = {};
    int dev = 0;
    if (hipError_t e = hipGetDevice(&dev); e != hipSuccess) return e;
    if (dev < 0 || dev >= 64 || granted_bytes[dev].load(std::memory_order_acquire) < pl.lds) {
      const hipError_t e =
          hipFuncSetAttribute((const void*)mfma_decode_general_kernel<ASYM, CH, T, MT, CPX, GM>,
                              hipFuncAttributeMaxDynamicSharedMemorySize, pl.lds);
      if (e != hipSuccess) return e;
      if (dev >= 0 && dev < 64) granted_bytes[dev].store(pl.lds, std::memory_order_release);
    }
    const int tiles = v.N / 16;
    const int sh = (v.gs & (v.gs - 1)) == 0 ? __builtin_ctz((unsigned)v.gs) : -1;
    const dim3 grid((unsigned)((tiles + T - 1) / T), (unsigned)((M + 16 * MT - 1) / (16 * MT)));
    mfma_decode_general_kernel<ASYM, CH, T, MT, CPX, GM><<<grid, DG_THREADS, pl.lds, s>>>(
        v.q, (const w4_half*)v.scales, v.zeros, x, c, v.N, v.K, v.gs, sh, v.G, M, tiles);
    return hipGetLastError();
  }
}

template <bool ASYM, int CH, int T, int MT, int CPX>
hipError_t general_go(const WView& v, const w4_half* x, w4_half* c, int M, hipStream_t s,
                      const GeneralPlan& pl) {
  if (v.gs >= 32) return general_gm<ASYM, CH, T, MT, CPX, 2>(v, x, c, M, s, pl);
  if constexpr (ASYM) {
    if (32 % v.gs == 0) return general_gm<ASYM, CH, T, MT, CPX, 1>(v, x, c, M, s, pl);
  }
  return general_gm<ASYM, CH, T, MT, CPX, 0>(v, x, c, M, s, pl);
}

template <bool ASYM, int CH, int T>
hipError_t general_mt(const WView& v, const w4_half* x, w4_half* c, int M, hipStream_t s,
                      const GeneralPlan& pl) {
  if (pl.mt == 1) {
    if constexpr (CH > 2) {
      if (pl.cpx == 2) return general_go<ASYM, CH, T, 1, 2>(v, x, c, M, s, pl);
    }
    return general_go<ASYM, CH, T, 1, 0>(v, x, c, M, s, pl);
  }
  if (pl.mt == 2) {
    if (pl.cpx == 1) return general_go<ASYM, CH, T, 2, 1>(v, x, c, M, s, pl);
    return general_go<ASYM, CH, T, 2, 0>(v, x, c, M, s, pl);
  }
  return general_go<ASYM, CH, T, 4, 0>(v, x, c, M, s, pl);
}

template <bool ASYM, int CH>
hipError_t general_t(const WView& v, const w4_half* x, w4_half* c, int M, hipStream_t s,
                     const GeneralPlan& pl) {
  switch (pl.t) {
    case 1: return general_mt<ASYM, CH, 1>(v, x, c, M, s, pl);
    case 2: return general_mt<ASYM, CH, 2>(v, x, c, M, s, pl);
    case 3: return general_mt<ASYM, CH, 3>(v, x, c, M, s, pl);
    default: return general_mt<ASYM, CH, 4>(v, x, c, M, s, pl);
  }
}

template <bool ASYM>
hipError_t general_ch(const WView& v, const w4_half* x, w4_half* c, int M, hipStream_t s,
                      const GeneralPlan& pl) {
  switch (pl.ch) {
    case 2: return general_t<ASYM, 2>(v, x, c, M, s, pl);
    case 3: return general_t<ASYM, 3>(v, x, c, M, s, pl);
    case 4: return general_t<ASYM, 4>(v, x, c, M, s, pl);
    default: return general_t<ASYM, 5>(v, x, c, M, s, pl);
  }
}

}  // namespace

bool decode_general_applies(const WView& v, const w4_half* x, const w4_half* c, int M) {
  GeneralPlan pl;
  return general_plan(v, x, c, M, &pl);
}

// Precondition: decode_general_applies(v, x, c, M); no hook.
hipError_t launch_decode_general(const WView& v, const w4_half* x, w4_half* c, int M, hipStream_t s) {
  GeneralPlan pl;
  if (!general_plan(v, x, c, M, &pl)) return hipErrorInvalidValue;
  return v.symmetric ? general_ch<false>(v, x, c, M, s, pl) : general_ch<true>(v, x, c, M, s, pl);
}

}  // namespace w4k
