// Split-S flash-decode phase 1 on the matrix cores, head dimension 128 or 64.
//
// A wave walks tiles of 32 cache positions.  Per tile:
//   scores   S[t][h] = sum_d K[t][d] q[h][d]  -- two groups of four
//            v_mfma_f32_16x16x32_f16, A = K rows (lane: position l%16, 32 of the
//            128 d), B = the query heads of the pass (up to 16 share one slab
//            read).  A lane's A operand is exactly what it loads: one dwordx4 of
//            packed codes (W4), two of bytes (FP8), four of halves (FP16); half of
//            that for D = 64, where a group is two MFMAs.
//   softmax  the result leaves lane (h = l%16, r = l/16) with the scores of head
//            h at positions {4r..4r+3, 16+4r..16+4r+3} of the tile; running
//            max / rescale are per lane, the tile max needs two lane exchanges.
//   output   O^T[d][h] += sum_t V[t][d] p[t][h]  -- eight MFMAs contracting over
//            the 32 positions, B = the probabilities straight from the score
//            registers (FP16), A = V transposed: lane (i = l%16, r = l/16) loads
//            the 8 cache elements d = 8i..8i+7 of its 8 positions (one packed
//            word, 8 bytes, or 16 bytes each) and expands them so that MFMA e
//            takes element e of every position: W4 expands two positions at a
//            time straight into that layout, FP16 / FP8 regroup the 8x8 block
//            with v_perm.  A ninth MFMA with A = 1 accumulates the denominators.
//            (D = 64 has only 8 element blocks for 16 operand rows: W4 lets lanes
//            i and i + 8 split the elements of block i % 8 -- 4 MFMAs --, FP16 /
//            FP8 repeat blocks 0..7 and drop the upper output rows.)
// Whole tiles are fetched with buffer loads whose wave-uniform part lives in the
// descriptor and the scalar offset; a ring of three raw tiles is refilled in
// place, two tiles in flight while one is computed.
// Dequantisation is the bit-exact register step of dq.cuh (the k_out / v_out
// hooks store those values); only the order of the FP32 sums differs from the
// vector kernel.  The four waves of a workgroup interleave tiles of one split
// and merge their (m, l, O) through LDS in wave order, so a split yields one
// partial and every sum has a fixed order: paged and contiguous caches give the
// same bytes.
#include <type_traits>

#include "dq.cuh"
#include "kernels.h"

namespace w4k {

constexpr int FM_TILE = 32;   // positions per wave tile
constexpr int FM_WAVES = 4;
constexpr int FM_DEPTH = 3;   // ring slots per wave: one tile computed, two in flight
constexpr int FM_HEADS = 16;  // query heads per pass

// What one lane fetches for one tile, before expansion.
// NC = D / 32: MFMAs per group of 16 positions = packed words (W4) per lane.
template <int KIND, int NC>
struct TileRaw;
template <int NC>
struct TileRaw<KIND_W4, NC> {
  uint32_t k[2][NC];
  _Float16 ks[2];
  uint32_t kz[2];
  uint32_t v[8], vz[8];
  _Float16 vs[8];
};
template <int NC>
struct TileRaw<KIND_F16, NC> {
  u4 k[2][NC];
  u4 v[8];
};
template <int NC>
struct TileRaw<KIND_F8, NC> {
  u2 k[2][NC];
  _Float16 ks[2];
  u2 v[8];
  _Float16 vs[8];
};

// Position of element e (0..7) of an expanded 8-element block: register and half.
template <int KIND>
__device__ __forceinline__ constexpr int reg_of(int e) {
  return KIND == KIND_W4 ? (e & 3) : KIND == KIND_F16 ? (e >> 1) : 2 * (e >> 2) + (e & 1);
}
template <int KIND>
__device__ __forceinline__ constexpr int half_of(int e) {
  return KIND == KIND_W4 ? (e >> 2) : KIND == KIND_F16 ? (e & 1) : ((e & 3) >> 1);
}
// Logical element held by (register p, half hf) of an expanded block.
template <int KIND>
__device__ __forceinline__ constexpr int elem_of(int p, int hf) {
  return KIND == KIND_W4 ? p + 4 * hf : KIND == KIND_F16 ? 2 * p + hf : 4 * (p >> 1) + (p & 1) + 2 * hf;
}

__device__ __forceinline__ h8 pack8(const h2 v[4]) {
  return h8{v[0][0], v[0][1], v[1][0], v[1][1], v[2][0], v[2][1], v[3][0], v[3][1]};
}

// PAGED: 0 contiguous slabs, 1 pages of a multiple of 16 rows (both halves of a
// tile lie in one page each), 2 any page size.  ALT: W4 with zero-points; FP8 with one
// scale per slab instead of one per row.
template <int KIND, int DH, bool HOOK, int PAGED, bool ALT>
__global__ __launch_bounds__(FM_WAVES * 64) void flash_mfma_phase1(const FlashArgs a,
                                                                   const int qh0,
                                                                   const int split_len,
                                                                   float* __restrict__ part) {
  constexpr bool ASYM = KIND == KIND_W4 && ALT, SLAB_SCALE = KIND == KIND_F8 && ALT;
  constexpr int FM_D = DH;       // head dimension
  constexpr int NC = DH / 32;    // MFMAs per score group; a lane's K slice is 8 * NC elements
  constexpr int NB = DH / 8;     // 8-element blocks per row
  constexpr int WD = DH / 8;     // packed words per W4 row
  constexpr int LDW = FM_D + 4;  // floats per (wave, head) merge row: O[D], l, m
  __shared__ float wo[FM_WAVES][FM_HEADS * LDW];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int c16 = lane & 15, q4 = lane >> 4;
  const int split = blockIdx.y, slab = blockIdx.x, nsplit = gridDim.y;  // slabs on x: no 65535 bound
  const int nh = min(FM_HEADS, a.group - qh0);
  const float inv_sqrt_d = 1.0f / sqrtf((float)FM_D);
  const float exp_scale = inv_sqrt_d * 1.44269504088896340736f;  // exp(x / sqrt(D)) = exp2(x * exp_scale)
  const int G = a.G, wg = words(a.G);
  const int vb = c16 & (NB - 1);                               // this lane's V element block
  const int gk = KIND == KIND_F16 ? 0 : (8 * NC * q4) / a.gs;  // group of this lane's K elements
  // First of the 8 row elements that score MFMA c contracts in this lane.  The
  // quantized kinds take a contiguous quarter of the row per lane (one load, one
  // scale).  FP16 needs a 16-byte load per MFMA either way, so there the four
  // k-blocks of an MFMA are neighbours: a load instruction reads 64 contiguous
  // bytes of each row instead of 16 bytes out of every 64.
  auto kcol = [&](int c) { return KIND == KIND_F16 ? 32 * c + 8 * q4 : 8 * NC * q4 + 8 * c; };
  const int gv = KIND == KIND_F16 ? 0 : (8 * vb) / a.gs;       // ... and of its V elements

  const int* bt = nullptr;
  long long rows0;
  if (PAGED) {
    bt = a.bt + (long long)(slab / a.Hkv) * a.bt_stride;
    rows0 = (long long)(slab % a.Hkv) * a.pool_rows;
  } else {
    rows0 = (long long)slab * a.S;
  }
  // Scales stay 16-bit values from the load to the packed operand: widened to 32
  // bits they would be masked right behind the load, which makes the wave wait
  // for a prefetch it has just issued.
  auto as_half = [](uint16_t b) { return __builtin_bit_cast(_Float16, b); };
  // Used where a prefetched scale is consumed: the empty statement keeps the
  // compiler from packing the scales of the next tile right behind their loads.
  auto at_use = [](_Float16 x) {
    asm("" : "+v"(x));
    return x;
  };
  _Float16 slab_sk = 0, slab_sv = 0;
  if (SLAB_SCALE) slab_sk = as_half(a.s_k[slab]), slab_sv = as_half(a.s_v[slab]);

  const int s0 = split * split_len;
  const int s1 = min(a.S, s0 + split_len);
  const long long hook_base = (long long)slab * a.S;
  const bool hook_k = HOOK && a.k_out && qh0 == 0, hook_v = HOOK && a.v_out && qh0 == 0;

  // Query operands: lane (head c16, k-block q4) of MFMA c holds
  // q[head][kcol(c) + elem_of(p, hf)].
  h8 qop[NC];
  {
    const uint16_t* qp =
        a.q + ((long long)slab * a.group + qh0 + min(c16, nh - 1)) * FM_D;
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      h2 t[4];
#pragma unroll
      for (int p = 0; p < 4; ++p) {
        const uint32_t lo = qp[kcol(c) + elem_of<KIND>(p, 0)], hi = qp[kcol(c) + elem_of<KIND>(p, 1)];
        t[p] = as_h2(c16 < nh ? (lo | (hi << 16)) : 0u);
      }
      qop[c] = pack8(t);
    }
  }

  // page of a position: a shift when the page size is a power of two (the scalar unit has
  // no divider: the quotient by a run-time page size is some twenty instructions, twice per tile)
  const int pshift = PAGED && (a.page & (a.page - 1)) == 0 ? __builtin_ctz((unsigned)a.page) : -1;
  auto page_of = [&](int t) { return pshift >= 0 ? t >> pshift : t / a.page; };
  // physical cache row of logical position t (t < S)
  auto phys = [&](int t, int pg_lo, long long base_lo, int pg_hi, long long base_hi, bool hi) -> long long {
    if (PAGED == 0) return rows0 + t;
    if (PAGED == 1) return (hi ? base_hi : base_lo) + (t - (hi ? pg_hi : pg_lo) * a.page);
    const int pg = page_of(t);
    return rows0 + (long long)bt[pg] * a.page + (t - pg * a.page);
  };

  // ---- whole tiles (all 32 positions below s1; with pages, each half of 16 in
  // one page): buffer loads whose wave-uniform part (slab base in the
  // descriptor, tile row in the scalar offset) never touches the vector ALU.
  // A lane adds only the constant byte offsets below.
  constexpr int ROWB = KIND == KIND_W4 ? DH / 2 : KIND == KIND_F8 ? DH : 2 * DH;  // bytes per cache row
  constexpr int VBB = ROWB / NB;                                                  // bytes per V block
  const long long slab_rows = PAGED ? a.pool_rows : a.S;
  // offsets are 32-bit: larger slabs take the general fetch for every tile
  const bool whole_ok = PAGED != 2 && slab_rows * ROWB < (1ll << 31) && slab_rows * G * 2 < (1ll << 31);
  auto rsrc = [&](const void* base, long long row_bytes) {
    const char* p0 = (const char*)base + rows0 * row_bytes;
    return __builtin_amdgcn_make_buffer_rsrc((void*)p0, 0, whole_ok ? (int)(slab_rows * row_bytes) : 0,
                                             0x00020000);
  };
  const auto rk = rsrc(a.k, ROWB), rv = rsrc(a.v, ROWB);
  const auto rsk = rsrc(a.s_k, 2 * G), rsv = rsrc(a.s_v, 2 * G);
  const auto rzk = rsrc(a.z_k, 4 * wg), rzv = rsrc(a.z_v, 4 * wg);
  const int kq_off = c16 * ROWB + q4 * (ROWB / 4);  // the lane's quarter of K row c16
  const int ks_off = 2 * (c16 * G + gk);
  const int kz_off = 4 * (c16 * wg + (gk >> 3));
  const int vq_off = 4 * q4 * ROWB + vb * VBB;      // block vb of the first of the lane's 4 V rows
  const int vs_off = 2 * (4 * q4 * G + gv);
  const int vz_off = 4 * (4 * q4 * wg + (gv >> 3));
  constexpr bool row_scales = KIND == KIND_W4 || (KIND == KIND_F8 && !SLAB_SCALE);

  // Row, in the slab (in the head's pool when paged), of position t, a multiple
  // of 16 that starts a half tile.  Positions past the last whole half are
  // clamped: the look-ahead below asks for them and drops the answer.
  auto slab_row = [&](int t) -> int {
    if (PAGED == 0) return t;
    const int tc = min(t, max(a.S - 16, 0));
    const int pg = page_of(tc);
    return bt[pg] * a.page + (tc - pg * a.page);
  };

  // rb[j]: slab_row(first position of half j)
  auto fetch_whole = [&](TileRaw<KIND, NC>& raw, const int rbs[2]) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int rb = rbs[j];
      constexpr int KQ = ROWB / 64;  // 16-byte pieces of a lane's K quarter (0: 8 bytes)
      u4 kraw[KQ ? KQ : 1];
      if constexpr (KQ == 0) {
        const u2 t2 = __builtin_amdgcn_raw_buffer_load_b64(rk, kq_off, rb * ROWB, 2);
        kraw[0] = u4{t2[0], t2[1], 0u, 0u};
      } else {
#pragma unroll
        for (int i = 0; i < KQ; ++i)
          kraw[i] = __builtin_amdgcn_raw_buffer_load_b128(
              rk, KIND == KIND_F16 ? c16 * ROWB + 2 * kcol(i) : kq_off + 16 * i, rb * ROWB, 2);
      }
      if constexpr (KIND == KIND_W4) {
#pragma unroll
        for (int c = 0; c < NC; ++c) raw.k[j][c] = kraw[0][c];
      } else if constexpr (KIND == KIND_F16) {
#pragma unroll
        for (int c = 0; c < NC; ++c) raw.k[j][c] = kraw[c];
      } else {
#pragma unroll
        for (int c = 0; c < NC; ++c) raw.k[j][c] = u2{kraw[c >> 1][2 * (c & 1)], kraw[c >> 1][2 * (c & 1) + 1]};
      }
      if constexpr (KIND != KIND_F16) {
        if (row_scales) raw.ks[j] = as_half(__builtin_amdgcn_raw_buffer_load_b16(rsk, ks_off, rb * 2 * G, 0));
        else raw.ks[j] = slab_sk;
      }
      if constexpr (KIND == KIND_W4)
        if (ASYM) raw.kz[j] = __builtin_amdgcn_raw_buffer_load_b32(rzk, kz_off, rb * 4 * wg, 0);
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int k = 4 * j + r;
        if constexpr (KIND == KIND_W4) {
          raw.v[k] = __builtin_amdgcn_raw_buffer_load_b32(rv, vq_off, (rb + r) * ROWB, 2);
          if (ASYM) raw.vz[k] = __builtin_amdgcn_raw_buffer_load_b32(rzv, vz_off, (rb + r) * 4 * wg, 0);
        } else if constexpr (KIND == KIND_F16) {
          raw.v[k] = __builtin_amdgcn_raw_buffer_load_b128(rv, vq_off, (rb + r) * ROWB, 2);
        } else {
          raw.v[k] = __builtin_amdgcn_raw_buffer_load_b64(rv, vq_off, (rb + r) * ROWB, 2);
        }
        if constexpr (KIND != KIND_F16) {
          if (row_scales) raw.vs[k] = as_half(__builtin_amdgcn_raw_buffer_load_b16(rsv, vs_off, (rb + r) * 2 * G, 0));
          else raw.vs[k] = slab_sv;
        }
      }
    }
  };

  auto fetch = [&](TileRaw<KIND, NC>& raw, int t0) {
    int pg_lo = 0, pg_hi = 0;
    long long base_lo = 0, base_hi = 0;
    if (PAGED == 1) {  // wave-uniform lookups: the page of each 16-position half
      pg_lo = page_of(min(t0, s1 - 1));
      pg_hi = page_of(min(t0 + 16, s1 - 1));
      base_lo = rows0 + (long long)bt[pg_lo] * a.page;
      base_hi = rows0 + (long long)bt[pg_hi] * a.page;
    }
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int t = min(t0 + 16 * j + c16, s1 - 1);
      const long long row = phys(t, pg_lo, base_lo, pg_hi, base_hi, j == 1);
      if constexpr (KIND == KIND_W4) {
        const uint32_t* src = (const uint32_t*)a.k + row * WD + NC * q4;
        if constexpr (NC == 4) {
          const u4 t4 = __builtin_nontemporal_load((const u4*)src);
#pragma unroll
          for (int c = 0; c < 4; ++c) raw.k[j][c] = t4[c];
        } else {
          const u2 t2 = __builtin_nontemporal_load((const u2*)src);
          raw.k[j][0] = t2[0];
          raw.k[j][1] = t2[1];
        }
        raw.ks[j] = as_half(a.s_k[row * G + gk]);
        if (ASYM) raw.kz[j] = a.z_k[row * wg + (gk >> 3)];
      } else if constexpr (KIND == KIND_F16) {
#pragma unroll
        for (int c = 0; c < NC; ++c)
          raw.k[j][c] = __builtin_nontemporal_load(
              (const u4*)((const uint16_t*)a.k + row * FM_D + kcol(c)));
      } else {
        const uint8_t* src = (const uint8_t*)a.k + row * FM_D + 8 * NC * q4;
        if constexpr (NC == 4) {
#pragma unroll
          for (int c = 0; c < 2; ++c) {
            const u4 t4 = __builtin_nontemporal_load((const u4*)(src + 16 * c));
            raw.k[j][2 * c] = u2{t4[0], t4[1]};
            raw.k[j][2 * c + 1] = u2{t4[2], t4[3]};
          }
        } else {
          const u4 t4 = __builtin_nontemporal_load((const u4*)src);
          raw.k[j][0] = u2{t4[0], t4[1]};
          raw.k[j][1] = u2{t4[2], t4[3]};
        }
        raw.ks[j] = SLAB_SCALE ? slab_sk : as_half(a.s_k[row * G + gk]);
      }
    }
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const int t = min(t0 + 16 * (k >> 2) + 4 * q4 + (k & 3), s1 - 1);
      const long long row = phys(t, pg_lo, base_lo, pg_hi, base_hi, k >= 4);
      if constexpr (KIND == KIND_W4) {
        raw.v[k] = __builtin_nontemporal_load((const uint32_t*)a.v + row * WD + vb);
        raw.vs[k] = as_half(a.s_v[row * G + gv]);
        if (ASYM) raw.vz[k] = a.z_v[row * wg + (gv >> 3)];
      } else if constexpr (KIND == KIND_F16) {
        raw.v[k] = __builtin_nontemporal_load((const u4*)((const uint16_t*)a.v + row * FM_D + 8 * vb));
      } else {
        raw.v[k] = __builtin_nontemporal_load((const u2*)((const uint8_t*)a.v + row * FM_D + 8 * vb));
        raw.vs[k] = SLAB_SCALE ? slab_sv : as_half(a.s_v[row * G + gv]);
      }
    }
  };

  // W4 at D = 64: a row has only 8 element blocks for the 16 operand rows of the
  // PV MFMA, so lanes i and i + 8 share block i % 8 and split its elements (0..3
  // and 4..7): 4 MFMAs whose row i is d = 8 (i % 8) + 4 (i / 8) + e, and half of
  // the expansion per lane.  (FP16 / FP8 at D = 64 repeat the blocks instead and
  // drop the upper rows.)
  constexpr bool SPLITV = KIND == KIND_W4 && DH == 64;
  constexpr int NE = SPLITV ? 4 : 8;  // PV MFMAs per tile = elements a lane expands per position
  const int hi8 = SPLITV ? c16 >> 3 : 0;
  f4 o[NE], lsum = f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int e = 0; e < NE; ++e) o[e] = f4{0.f, 0.f, 0.f, 0.f};
  float m_run = -INFINITY;
  const h8 ones = h8{1, 1, 1, 1, 1, 1, 1, 1};

  auto store16 = [&](uint16_t* dst, const h2 nat[4]) {
    *(u4*)dst = u4{as_u32(nat[0]), as_u32(nat[1]), as_u32(nat[2]), as_u32(nat[3])};
  };

  // whole: every position of the tile is below s1 (no masking)
  auto compute = [&](const TileRaw<KIND, NC>& raw, int t0, auto whole) {
    constexpr bool WHOLE = decltype(whole)::value;
    // ---- scores
    f4 sc[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      sc[j] = f4{0.f, 0.f, 0.f, 0.f};
      const int t = t0 + 16 * j + c16;
      uint16_t* kdst = HOOK ? a.k_out + (hook_base + t) * FM_D : nullptr;
      const bool kst = hook_k && t < s1;
      _Float16 ksc = 0;
      if constexpr (KIND != KIND_F16) ksc = at_use(raw.ks[j]);
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        h2 d[4];
        if constexpr (KIND == KIND_W4) {
          const int z = ASYM ? (int)((raw.kz[j] >> (4 * (gk & 7))) & 0xFu) : 8;
          dq_w4(raw.k[j][c], w4_group(ksc, z), d);
          if (kst) {
            h2 nat[4];
            to_natural(d, nat);
            store16(kdst + kcol(c), nat);
          }
        } else if constexpr (KIND == KIND_F16) {
#pragma unroll
          for (int p = 0; p < 4; ++p) d[p] = as_h2(raw.k[j][c][p]);
          if (kst) store16(kdst + kcol(c), d);
        } else {
          const h2 s = splat(ksc);
          dq_f8(raw.k[j][c][0], s, d);
          dq_f8(raw.k[j][c][1], s, d + 2);
          if (kst) {
            h2 nat[4];
            to_natural_f8(d, nat);
            to_natural_f8(d + 2, nat + 2);
            store16(kdst + kcol(c), nat);
          }
        }
        sc[j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pack8(d), qop[c], sc[j], 0, 0, 0);
      }
    }
    // ---- online softmax for head c16 over this lane's 8 positions.  The running
    // maximum is kept on the raw dot products (the scale is positive, so the order
    // is the same); exp((x - m) / sqrt(D)) is one FMA and one v_exp_f32.
    float x[8];
    float tmax = -INFINITY;
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const int t = t0 + 16 * (k >> 2) + 4 * q4 + (k & 3);
      x[k] = WHOLE || t < s1 ? sc[k >> 2][k & 3] : -INFINITY;
      tmax = fmaxf(tmax, x[k]);
    }
    tmax = fmaxf(tmax, __shfl_xor(tmax, 16, 64));
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
    const float m_new = fmaxf(m_run, tmax);
    const float m_use = m_new == -INFINITY ? 0.0f : m_new;
    if (__builtin_amdgcn_ballot_w64(m_new > m_run) != 0) {  // wave-uniform
      const float alpha = __builtin_amdgcn_exp2f((m_run - m_use) * exp_scale);
#pragma unroll
      for (int e = 0; e < NE; ++e) o[e] *= alpha;
      lsum *= alpha;
    }
    m_run = m_new;
    const float m_sub = -m_use * exp_scale;
    h2 pr[4];
#pragma unroll
    for (int k = 0; k < 4; ++k)
      pr[k] = h2{(_Float16)__builtin_amdgcn_exp2f(__builtin_fmaf(x[2 * k], exp_scale, m_sub)),
                 (_Float16)__builtin_amdgcn_exp2f(__builtin_fmaf(x[2 * k + 1], exp_scale, m_sub))};
    const h8 pop = pack8(pr);
    lsum = __builtin_amdgcn_mfma_f32_16x16x32_f16(ones, pop, lsum, 0, 0, 0);
    // ---- V: expand the 8 positions x 8 elements of this lane so that MFMA e takes
    // element e of every position, accumulate
    auto hook_store_v = [&](int k, const h2 nat[4]) {
      const int t = t0 + 16 * (k >> 2) + 4 * q4 + (k & 3);
      if (hook_v && t < s1 && c16 < NB) store16(a.v_out + (hook_base + t) * FM_D + 8 * vb, nat);
    };
    // the 4 elements of a lane of the split layout
    auto hook_store_v4 = [&](int k, const h2 nat[2]) {
      const int t = t0 + 16 * (k >> 2) + 4 * q4 + (k & 3);
      if (hook_v && t < s1)
        *(u2*)(a.v_out + (hook_base + t) * FM_D + 8 * vb + 4 * hi8) = u2{as_u32(nat[0]), as_u32(nat[1])};
    };
    if constexpr (KIND == KIND_W4) {
      // Two positions at a time: v_perm puts byte b of both words into the two
      // halves of a register, so each expanded register already is the pair
      // (position 2 kk, position 2 kk + 1) of one element -- the MFMA operand
      // layout -- and the two scales ride in one packed multiply.  Per element the
      // arithmetic is that of dq_w4: (1024 + n) - (1024 + z) or (64 + n) - (64 + z),
      // exact, then one rounding in the multiply by the scale.
      h2 pe[4][NE];
      uint32_t magic_lo = 0x64006400u, magic_hi = 0x54005400u;
      asm("" : "+v"(magic_lo));
      asm("" : "+v"(magic_hi));
      // byte b of a lane's share of the word is byte b + 2 hi8 of the word
      const uint32_t byte0 = 2u * (uint32_t)hi8;
#pragma unroll
      for (int kk = 0; kk < 4; ++kk) {
        const uint32_t w0 = raw.v[2 * kk], w1 = raw.v[2 * kk + 1];
        const h2 s2 = h2{at_use(raw.vs[2 * kk]), at_use(raw.vs[2 * kk + 1])};
        uint32_t zz = 0x00080008u;  // zero points of the two positions, one per half
        if (ASYM) {
          const int sh = 4 * (gv & 7);
          zz = ((raw.vz[2 * kk] >> sh) & 0xFu) | (((raw.vz[2 * kk + 1] >> sh) & 0xFu) << 16);
        }
        const h2 clo = as_h2(0xE400E400u | zz);         // -(1024 + z), ulp 1
        const h2 chi = as_h2(0xD400D400u | (zz << 4));  // -(64 + z), ulp 1/16
#pragma unroll
        for (int b = 0; b < NE / 2; ++b) {
          const uint32_t p = __builtin_amdgcn_perm(w1, w0, 0x0c000c00u | ((4u + b + byte0) << 16) | (b + byte0));
          pe[kk][2 * b] = (as_h2(and_or(p, 0x000F000Fu, magic_lo)) + clo) * s2;
          pe[kk][2 * b + 1] = (as_h2(and_or(p, 0x00F000F0u, magic_hi)) + chi) * s2;
        }
        if constexpr (HOOK) {
          h2 n0[4], n1[4];
#pragma unroll
          for (int i = 0; i < NE / 2; ++i) {
            n0[i] = as_h2(__builtin_amdgcn_perm(as_u32(pe[kk][2 * i + 1]), as_u32(pe[kk][2 * i]), 0x05040100u));
            n1[i] = as_h2(__builtin_amdgcn_perm(as_u32(pe[kk][2 * i + 1]), as_u32(pe[kk][2 * i]), 0x07060302u));
          }
          if constexpr (SPLITV) {
            hook_store_v4(2 * kk, n0);
            hook_store_v4(2 * kk + 1, n1);
          } else {
            hook_store_v(2 * kk, n0);
            hook_store_v(2 * kk + 1, n1);
          }
        }
      }
#pragma unroll
      for (int e = 0; e < NE; ++e) {
        const h2 at[4] = {pe[0][e], pe[1][e], pe[2][e], pe[3][e]};
        o[e] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pack8(at), pop, o[e], 0, 0, 0);
      }
    } else {
      h2 vt[8][4];
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        if constexpr (KIND == KIND_F16) {
#pragma unroll
          for (int p = 0; p < 4; ++p) vt[k][p] = as_h2(raw.v[k][p]);
          if constexpr (HOOK) hook_store_v(k, vt[k]);
        } else {
          const h2 s = splat(at_use(raw.vs[k]));
          dq_f8(raw.v[k][0], s, vt[k]);
          dq_f8(raw.v[k][1], s, vt[k] + 2);
          if constexpr (HOOK) {
            h2 nat[4];
            to_natural_f8(vt[k], nat);
            to_natural_f8(vt[k] + 2, nat + 2);
            hook_store_v(k, nat);
          }
        }
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        constexpr uint32_t LO = 0x05040100u, HI = 0x07060302u;
        const int rg = reg_of<KIND>(e);
        const uint32_t sel = half_of<KIND>(e) ? HI : LO;
        h2 at[4];
#pragma unroll
        for (int kk = 0; kk < 4; ++kk)
          at[kk] = as_h2(__builtin_amdgcn_perm(as_u32(vt[2 * kk + 1][rg]), as_u32(vt[2 * kk][rg]), sel));
        o[e] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pack8(at), pop, o[e], 0, 0, 0);
      }
    }
  };

  // tiles of this wave: s0 + 32 * (wave + 4 * it)
  const int nit = (s1 - s0 + FM_WAVES * FM_TILE - 1) / (FM_WAVES * FM_TILE);
  auto tile_start = [&](int it) { return s0 + FM_TILE * (wave + FM_WAVES * it); };
  // the first nwhole tiles of this wave lie wholly below s1
  const int room = s1 - s0 - FM_TILE * (wave + 1);
  const int nwhole = whole_ok && room >= 0 ? room / (FM_WAVES * FM_TILE) + 1 : 0;
  // Tile number `it` of this wave into `raw`: buffer loads when it is whole, the
  // general fetch when it is cut by s1, nothing when it lies past the split.
  auto fetch_any = [&](TileRaw<KIND, NC>& raw, int it) {
    if (it < nwhole) {
      const int rb[2] = {slab_row(tile_start(it)), slab_row(tile_start(it) + 16)};
      fetch_whole(raw, rb);
    } else if (it < nit) {
      fetch(raw, tile_start(it));
    }
  };
  // A ring slot is refilled right after the tile in it has been consumed, into
  // the same registers: the loop carries no copies, and DEPTH - 1 tiles are in
  // flight while one is computed.
  // (FP8 with row scales: two slots keep two waves per SIMD resident, which pays there)
  constexpr int DEPTH = KIND == KIND_F8 && !SLAB_SCALE ? 2 : FM_DEPTH;
  TileRaw<KIND, NC> ring[DEPTH];
#pragma unroll
  for (int d = 0; d < DEPTH; ++d) fetch_any(ring[d], d);
  int it0 = 0;
  // Page-table lookups run one tile ahead of the loads that need them, so the
  // scalar load's latency is off the path to the vector loads.
  int rb_next[2] = {slab_row(tile_start(DEPTH)), slab_row(tile_start(DEPTH) + 16)};
  for (; it0 + 2 * DEPTH <= nwhole; it0 += DEPTH) {  // computes and fetches whole tiles only
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      compute(ring[d], tile_start(it0 + d), std::true_type{});
      __builtin_amdgcn_sched_barrier(0);
      const int rb[2] = {rb_next[0], rb_next[1]};
      const int t_after = tile_start(it0 + d + DEPTH + 1);
      rb_next[0] = slab_row(t_after);
      rb_next[1] = slab_row(t_after + 16);
      fetch_whole(ring[d], rb);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  for (; it0 < nit; it0 += DEPTH) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      if (it0 + d < nit) compute(ring[d], tile_start(it0 + d), std::false_type{});
      __builtin_amdgcn_sched_barrier(0);
      fetch_any(ring[d], it0 + d + DEPTH);
      __builtin_amdgcn_sched_barrier(0);
    }
  }

  // ---- merge the four waves in wave order: lane (head c16, q4) holds
  // O[head][32 q4 + 8 r + e] in o[e][r] (output rows past D / 8 are repeats: dropped)
  float* mine = wo[wave] + c16 * LDW;
#pragma unroll
  for (int e = 0; e < NE; ++e)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int i = 4 * q4 + r;  // operand row of the PV MFMA
      if constexpr (SPLITV) mine[8 * (i & 7) + 4 * (i >> 3) + e] = o[e][r];
      else if (i < NB) mine[8 * i + e] = o[e][r];
    }
  if (q4 == 0) {
    mine[FM_D] = lsum[0];
    mine[FM_D + 1] = m_run * inv_sqrt_d;  // the maximum of the scaled scores
  }
  __syncthreads();
  if (nsplit == 1) {
    // One split per slab (short caches): no partials and no second launch.  The value
    // is the one the merge kernel gives for a single split, sum * (1 / l).
    for (int i = threadIdx.x; i < nh * FM_D; i += FM_WAVES * 64) {
      const int h = i / FM_D, j = i - h * FM_D;
      float mw[FM_WAVES], M = -INFINITY;
#pragma unroll
      for (int w = 0; w < FM_WAVES; ++w) {
        mw[w] = wo[w][h * LDW + FM_D + 1];
        M = fmaxf(M, mw[w]);
      }
      float sum = 0.0f, l = 0.0f;
#pragma unroll
      for (int w = 0; w < FM_WAVES; ++w) {
        const float e = __expf(mw[w] - M);
        sum += e * wo[w][h * LDW + j];
        l += e * wo[w][h * LDW + FM_D];
      }
      const _Float16 hv = (_Float16)(sum * (1.0f / l));
      a.out[((long long)slab * a.group + qh0 + h) * FM_D + j] = __builtin_bit_cast(uint16_t, hv);
    }
    return;
  }
  for (int i = threadIdx.x; i < nh * (FM_D + 1); i += FM_WAVES * 64) {
    const int h = i / (FM_D + 1), j = i - h * (FM_D + 1);  // j < 128: O[j]; j == 128: l
    float mw[FM_WAVES], M = -INFINITY;
#pragma unroll
    for (int w = 0; w < FM_WAVES; ++w) {
      mw[w] = wo[w][h * LDW + FM_D + 1];
      M = fmaxf(M, mw[w]);
    }
    float sum = 0.0f;
#pragma unroll
    for (int w = 0; w < FM_WAVES; ++w) sum += __expf(mw[w] - M) * wo[w][h * LDW + j];
    float* dst = part + (((long long)slab * a.group + qh0 + h) * nsplit + split) * (FM_D + 2);
    if (j < FM_D) {
      dst[2 + j] = sum;
    } else {
      dst[1] = sum;
      dst[0] = M;
    }
  }
}

template <int KIND, bool HOOK, int PAGED>
static hipError_t go_asym(const FlashArgs& a, int qh0, const FlashPlan& pl, float* part,
                          hipStream_t s) {
  const dim3 grid((unsigned)a.H, (unsigned)pl.nsplit);
  const bool asym = (KIND == KIND_W4 && !a.symmetric) || (KIND == KIND_F8 && a.scale_mode == 1);
#define W4_GO(DH, ASYM) \
  flash_mfma_phase1<KIND, DH, HOOK, PAGED, ASYM><<<grid, FM_WAVES * 64, 0, s>>>(a, qh0, pl.split_len, part)
  if (a.D == 128) {
    if (asym) W4_GO(128, true); else W4_GO(128, false);
  } else {
    if (asym) W4_GO(64, true); else W4_GO(64, false);
  }
#undef W4_GO
  return hipGetLastError();
}

template <int KIND>
static hipError_t go_kind(const FlashArgs& a, int qh0, const FlashPlan& pl, float* part,
                          hipStream_t s) {
  const bool hook = a.k_out || a.v_out;
  if constexpr (KIND == KIND_W4) {
    if (a.bt) {
      if (a.page % 16 == 0)
        return hook ? go_asym<KIND, true, 1>(a, qh0, pl, part, s) : go_asym<KIND, false, 1>(a, qh0, pl, part, s);
      return hook ? go_asym<KIND, true, 2>(a, qh0, pl, part, s) : go_asym<KIND, false, 2>(a, qh0, pl, part, s);
    }
  }
  return hook ? go_asym<KIND, true, 0>(a, qh0, pl, part, s) : go_asym<KIND, false, 0>(a, qh0, pl, part, s);
}

bool flash_mfma_applies(const FlashArgs& a) {
  if (a.D != 128 && a.D != 64) return false;
  // one group per lane's K slice (32 elements at D = 128, 16 at D = 64) and per 8-element V block
  if (a.kind != KIND_F16 && a.gs % (a.D / 4)) return false;
  return ((((uintptr_t)a.k | (uintptr_t)a.v) & 15) == 0) &&
         ((((uintptr_t)a.k_out | (uintptr_t)a.v_out) & 15) == 0);
}

bool try_flash_mfma(const FlashArgs& a, const FlashPlan& pl, float* part, hipStream_t s,
                    hipError_t* err) {
  if (!flash_mfma_applies(a) || pl.split_len % (FM_WAVES * FM_TILE)) return false;
  *err = hipSuccess;
  for (int qh0 = 0; qh0 < a.group && *err == hipSuccess; qh0 += FM_HEADS) {
    if (a.kind == KIND_F16) *err = go_kind<KIND_F16>(a, qh0, pl, part, s);
    else if (a.kind == KIND_W4) *err = go_kind<KIND_W4>(a, qh0, pl, part, s);
    else *err = go_kind<KIND_F8>(a, qh0, pl, part, s);
  }
  return true;
}

}  // namespace w4k
