// Split-S flash-decode attention over FP16, W4, FP8-E4M3 and paged-W4 caches.
//
// One query token per head.  A cache "slab" is one (sequence, kv-head) pair:
// S rows of D elements; `group` query heads read the same slab (grouped-query
// attention), so the slab is streamed from HBM once for all of them.
//
// Phase 1: grid (slab, split).  A workgroup walks its split of the sequence in
// tiles of 256 positions: K pass -> scaled scores in LDS, tile max, then V pass
// accumulating exp(s - m) * v in FP32 registers; a running (m, l, acc) is
// rescaled once per tile.  Lanes own a fixed slice of D (E elements) and a
// position slot, so a wave-load is a contiguous 1 KiB of cache rows (dwordx4
// per lane).  Cache elements are expanded in VGPRs with the bit-exact steps of
// dq.cuh; the k_out / v_out hooks store exactly those values.
// Phase 2: one workgroup per query head combines the per-split partials
// (m, l, acc[D]) in split order.  Every reduction has a fixed order, so
// results are reproducible bit for bit (the paged kernel equals the
// contiguous one exactly).
#include "dq.cuh"
#include "kernels.h"

namespace w4k {

constexpr int FL_TILE = 256;   // positions per tile
constexpr int FL_WAVES = 4;


// Offset within a lane's E-element chunk of register pair p, half hf.
template <int KIND>
__device__ __forceinline__ constexpr int d_of(int p, int hf) {
  if (KIND == KIND_F16) return 2 * p + hf;
  if (KIND == KIND_W4) return 8 * (p >> 2) + (p & 3) + 4 * hf;  // (i, i+4) per word
  return 4 * (p >> 1) + (p & 1) + 2 * hf;                        // (b0,b2),(b1,b3)
}

struct RowSrc {
  const void* data;       // cache elements of this slab side
  const uint16_t* scale;  // per (row, group) scales (W4, FP8 mode 0)
  const uint32_t* zero;   // W4 asymmetric
  uint32_t slab_scale;    // FP8 mode 1: scale bits for the whole slab
};

// Load the lane's chunk [dbase, dbase+E) of cache row `row` and expand it to
// E/2 packed halves in register order.  Elements at d >= D are unspecified but
// finite (they meet zero query / are never stored).
template <int KIND, int E, bool FASTLD>
__device__ __forceinline__ void load_chunk(const RowSrc& src, const FlashArgs& a,
                                           long long row, int dbase, h2* v) {
  if constexpr (KIND == KIND_F16) {
    const uint16_t* p = (const uint16_t*)src.data + row * a.D + dbase;
    u4 t = {0u, 0u, 0u, 0u};
    if (FASTLD) {
      t = __builtin_nontemporal_load((const u4*)p);
    } else {
      uint16_t e[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) e[j] = (dbase + j < a.D) ? p[j] : (uint16_t)0;
      t = u4{e[0] | ((uint32_t)e[1] << 16), e[2] | ((uint32_t)e[3] << 16),
             e[4] | ((uint32_t)e[5] << 16), e[6] | ((uint32_t)e[7] << 16)};
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = as_h2(t[i]);
  } else if constexpr (KIND == KIND_W4) {
    const int wd = words(a.D);
    const uint32_t* p = (const uint32_t*)src.data + row * wd + (dbase >> 3);
    constexpr int NW = E / 8;
    uint32_t w[NW];
    if constexpr (NW == 4) {
      const u4 t = __builtin_nontemporal_load((const u4*)p);
#pragma unroll
      for (int j = 0; j < 4; ++j) w[j] = t[j];
    } else {
      w[0] = (dbase < a.D) ? p[0] : 0u;
    }
    const int wg = words(a.G);
#pragma unroll
    for (int j = 0; j < NW; ++j) {
      const int g = min((dbase + 8 * j) / a.gs, a.G - 1);
      const int z = a.symmetric ? 8
                                : (int)((src.zero[row * wg + (g >> 3)] >> (4 * (g & 7))) & 0xF);
      dq_w4(w[j], w4_group(src.scale[row * a.G + g], z), v + 4 * j);
    }
  } else {
    const uint8_t* p = (const uint8_t*)src.data + row * a.D + dbase;
    constexpr int NW = E / 4;
    uint32_t w[NW];
    if constexpr (NW == 4) {
      const u4 t = __builtin_nontemporal_load((const u4*)p);
#pragma unroll
      for (int j = 0; j < 4; ++j) w[j] = t[j];
    } else {
#pragma unroll
      for (int j = 0; j < NW; ++j) w[j] = (dbase + 4 * j < a.D) ? ((const uint32_t*)p)[j] : 0u;
    }
#pragma unroll
    for (int j = 0; j < NW; ++j) {
      uint32_t sb = src.slab_scale;
      if (a.scale_mode == 0) {
        const int g = min((dbase + 4 * j) / a.gs, a.G - 1);
        sb = src.scale[row * a.G + g];
      }
      dq_f8(w[j], splat_bits(sb), v + 2 * j);
    }
  }
}

// Store the chunk's dequantized halves to the hook buffer in logical order.
template <int KIND, int E>
__device__ __forceinline__ void store_hook(uint16_t* dst, int dbase, int D, const h2* v) {
#pragma unroll
  for (int p = 0; p < E / 2; ++p)
#pragma unroll
    for (int hf = 0; hf < 2; ++hf) {
      const int d = dbase + d_of<KIND>(p, hf);
      if (d < D) {
        const uint32_t pair = as_u32(v[p]);
        dst[d] = (uint16_t)(hf ? pair >> 16 : pair & 0xFFFFu);
      }
    }
}

// Physical cache row of logical position t.
__device__ __forceinline__ long long phys_row(const FlashArgs& a, const int* bt,
                                              long long slab_rows0, int t) {
  if (bt == nullptr) return slab_rows0 + t;
  const int pg = t / a.page;
  return slab_rows0 + (long long)bt[pg] * a.page + (t - pg * a.page);
}

template <int KIND, int E, int GQ, bool HOOK, bool FASTLD>
__global__ __launch_bounds__(FL_WAVES * 64) void flash_phase1(const FlashArgs a,
                                                              const int qh0, const int LP,
                                                              const int split_len,
                                                              float* __restrict__ part) {
  __shared__ float sc[GQ][FL_TILE];
  __shared__ float wred[FL_WAVES][GQ][512 + 2];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int split = blockIdx.y, slab = blockIdx.x;  // slabs on x: no 65535 bound
  const int nsplit = gridDim.y;
  const int PW = 64 / LP;             // position slots per wave
  const int sub = lane & (LP - 1);    // which E-chunk of the row
  const int slot = lane / LP;
  const int dbase = sub * E;
  const bool chunk_ok = dbase < a.D;
  const int D = a.D;
  const float inv_sqrt_d = 1.0f / sqrtf((float)D);

  // cache addressing
  const int* bt = nullptr;
  long long rows0;
  if (a.bt) {
    bt = a.bt + (long long)(slab / a.Hkv) * a.bt_stride;
    rows0 = (long long)(slab % a.Hkv) * a.pool_rows;
  } else {
    rows0 = (long long)slab * a.S;
  }
  RowSrc ks{a.k, a.s_k, a.z_k, 0u}, vs{a.v, a.s_v, a.z_v, 0u};
  if (KIND == KIND_F8 && a.scale_mode == 1) {
    ks.slab_scale = a.s_k[slab];
    vs.slab_scale = a.s_v[slab];
  }

  // this pass's query heads, in register order
  h2 qv[GQ][E / 2];
#pragma unroll
  for (int h = 0; h < GQ; ++h) {
    const uint16_t* qp = a.q + ((long long)slab * a.group + qh0 + h) * D;
#pragma unroll
    for (int p = 0; p < E / 2; ++p) {
      const int d0 = dbase + d_of<KIND>(p, 0), d1 = dbase + d_of<KIND>(p, 1);
      const uint32_t lo = d0 < D ? qp[d0] : 0u, hi = d1 < D ? qp[d1] : 0u;
      qv[h][p] = as_h2(lo | (hi << 16));
    }
  }

  float acc[GQ][E];
  float m_run[GQ], l_run[GQ];
#pragma unroll
  for (int h = 0; h < GQ; ++h) {
    m_run[h] = -INFINITY;
    l_run[h] = 0.0f;
#pragma unroll
    for (int e = 0; e < E; ++e) acc[h][e] = 0.0f;
  }

  const int s0 = split * split_len;
  const int s1 = min(a.S, s0 + split_len);
  const long long hook_base = (long long)slab * a.S;

  for (int t0 = s0; t0 < s1; t0 += FL_TILE) {
    const int t1 = min(s1, t0 + FL_TILE);
    // ---- K pass: scaled scores of the tile into LDS
    for (int tb = t0 + wave * PW; tb < t1; tb += FL_WAVES * PW) {
      const int t = tb + slot;
      const bool live = t < t1 && chunk_ok;
      float s[GQ];
#pragma unroll
      for (int h = 0; h < GQ; ++h) s[h] = 0.0f;
      if (live) {
        h2 kv[E / 2];
        load_chunk<KIND, E, FASTLD>(ks, a, phys_row(a, bt, rows0, t), dbase, kv);
        if (HOOK && a.k_out && qh0 == 0)
          store_hook<KIND, E>(a.k_out + (hook_base + t) * D, dbase, D, kv);
#pragma unroll
        for (int h = 0; h < GQ; ++h)
#pragma unroll
          for (int p = 0; p < E / 2; ++p) s[h] = dot2(kv[p], qv[h][p], s[h]);
      }
#pragma unroll
      for (int h = 0; h < GQ; ++h) {
        for (int off = 1; off < LP; off <<= 1) s[h] += __shfl_xor(s[h], off, 64);
        if (sub == 0 && t < t1) sc[h][t - t0] = s[h] * inv_sqrt_d;
      }
    }
    __syncthreads();
    // ---- tile max (every wave computes it; no second barrier needed)
    float m_new[GQ];
#pragma unroll
    for (int h = 0; h < GQ; ++h) {
      float m = -INFINITY;
      for (int i = lane; i < t1 - t0; i += 64) m = fmaxf(m, sc[h][i]);
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) m = fmaxf(m, __shfl_xor(m, off, 64));
      m_new[h] = fmaxf(m_run[h], m);
      const float r = __expf(m_run[h] - m_new[h]);  // 0 on the first tile
      l_run[h] *= r;
#pragma unroll
      for (int e = 0; e < E; ++e) acc[h][e] *= r;
      m_run[h] = m_new[h];
    }
    // ---- V pass
    for (int tb = t0 + wave * PW; tb < t1; tb += FL_WAVES * PW) {
      const int t = tb + slot;
      if (t < t1 && chunk_ok) {
        h2 vv[E / 2];
        load_chunk<KIND, E, FASTLD>(vs, a, phys_row(a, bt, rows0, t), dbase, vv);
        if (HOOK && a.v_out && qh0 == 0)
          store_hook<KIND, E>(a.v_out + (hook_base + t) * D, dbase, D, vv);
#pragma unroll
        for (int h = 0; h < GQ; ++h) {
          const float p = __expf(sc[h][t - t0] - m_new[h]);
          l_run[h] += p;
#pragma unroll
          for (int i = 0; i < E / 2; ++i) {
            acc[h][2 * i] = fmaf(p, (float)vv[i][0], acc[h][2 * i]);
            acc[h][2 * i + 1] = fmaf(p, (float)vv[i][1], acc[h][2 * i + 1]);
          }
        }
      }
    }
    __syncthreads();  // sc is rewritten by the next tile
  }

  // ---- combine the position slots of a wave, then the waves, in fixed order
#pragma unroll
  for (int h = 0; h < GQ; ++h) {
    for (int off = LP; off < 64; off <<= 1) {
      l_run[h] += __shfl_xor(l_run[h], off, 64);
#pragma unroll
      for (int e = 0; e < E; ++e) acc[h][e] += __shfl_xor(acc[h][e], off, 64);
    }
    if (slot == 0) {
      if (chunk_ok) {
#pragma unroll
        for (int p = 0; p < E / 2; ++p)
#pragma unroll
          for (int hf = 0; hf < 2; ++hf) {
            const int d = dbase + d_of<KIND>(p, hf);
            if (d < D) wred[wave][h][2 + d] = acc[h][2 * p + hf];
          }
      }
      if (sub == 0) wred[wave][h][1] = l_run[h];
    }
  }
  __syncthreads();
  for (int i = threadIdx.x; i < GQ * (D + 1); i += FL_WAVES * 64) {
    const int h = i / (D + 1), j = 1 + (i - h * (D + 1));  // j = 1: l, else acc[j-2]
    const float sum = ((wred[0][h][j] + wred[1][h][j]) + wred[2][h][j]) + wred[3][h][j];
    float* dst = part + (((long long)slab * a.group + qh0 + h) * nsplit + split) * (D + 2);
    dst[j] = sum;
    if (j == 1) dst[0] = m_run[h];
  }
}

// Phase 2: out[d] = sum_t exp(m_t - M) acc_t[d] / sum_t exp(m_t - M) l_t.
// One workgroup per query head.  The split weights are computed once, in
// parallel over t, and kept in LDS; the sum over t for each d is cut into up to
// four runs of consecutive t handled by different threads and added in run
// order.  Every reduction is a fixed tree, so the result depends only on the
// partials.
constexpr int P2_THREADS = 256;
constexpr int P2_MAXT = 2048;  // flash_plan never makes more splits

__device__ __forceinline__ float block_reduce(float v, float* tmp, bool is_max) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const float o = __shfl_xor(v, off, 64);
    v = is_max ? fmaxf(v, o) : v + o;
  }
  const int wave = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) tmp[wave] = v;
  __syncthreads();
  float r = tmp[0];
#pragma unroll
  for (int w = 1; w < P2_THREADS / 64; ++w) r = is_max ? fmaxf(r, tmp[w]) : r + tmp[w];
  __syncthreads();
  return r;
}

__global__ __launch_bounds__(P2_THREADS) void flash_phase2(const float* __restrict__ part,
                                                           w4_half* __restrict__ out,
                                                           const int T, const int D) {
  __shared__ float wts[P2_MAXT];
  __shared__ float tmp[P2_THREADS / 64];
  __shared__ float runs[3][256];
  const long long hq = blockIdx.x;
  const int stride = D + 2;
  const float* hb = part + hq * T * stride;
  float m = -INFINITY;
  for (int t = threadIdx.x; t < T; t += P2_THREADS) m = fmaxf(m, hb[(long long)t * stride]);
  const float M = block_reduce(m, tmp, true);
  float den = 0.0f;
  for (int t = threadIdx.x; t < T; t += P2_THREADS) {
    const float w = __expf(hb[(long long)t * stride] - M);
    wts[t] = w;
    den += w * hb[(long long)t * stride + 1];
  }
  den = block_reduce(den, tmp, false);  // also orders the wts writes before the reads below
  const float inv = 1.0f / den;
  const int dpad = (D + 63) & ~63;
  if (dpad <= 256) {
    const int nrun = P2_THREADS / dpad;  // 4, 2 or 1 runs of consecutive t
    const int run = threadIdx.x / dpad, d = threadIdx.x - run * dpad;
    const int per = (T + nrun - 1) / nrun;
    const int ta = min(T, run * per), tb = min(T, ta + per);
    float acc = 0.0f;
    if (run < nrun && d < D) {
#pragma unroll 4
      for (int t = ta; t < tb; ++t) acc += wts[t] * hb[(long long)t * stride + 2 + d];
    }
    if (run > 0 && run < nrun && d < D) runs[run - 1][d] = acc;
    __syncthreads();
    if (run == 0 && d < D) {
      for (int r = 1; r < nrun; ++r) acc += runs[r - 1][d];
      const _Float16 h = (_Float16)(acc * inv);
      out[hq * D + d] = __builtin_bit_cast(uint16_t, h);
    }
  } else {
    for (int d = threadIdx.x; d < D; d += P2_THREADS) {
      float acc = 0.0f;
#pragma unroll 4
      for (int t = 0; t < T; ++t) acc += wts[t] * hb[(long long)t * stride + 2 + d];
      const _Float16 h = (_Float16)(acc * inv);
      out[hq * D + d] = __builtin_bit_cast(uint16_t, h);
    }
  }
}

// ---- host side -------------------------------------------------------------

FlashPlan flash_plan(const FlashArgs& a) {
  // Enough workgroups to fill 256 CUs, but splits no shorter than one tile; a
  // longer split writes fewer partials.  Measured at 64 slabs x 32768 positions:
  // the matrix-core kernel is fastest with 2 workgroups per CU (512 in all; 256,
  // 768, 1024, 2048 and 4096 were slower), the vector kernel with 8.
  const int tiles = (a.S + FL_TILE - 1) / FL_TILE;
  const int per_cu = flash_mfma_applies(a) ? 2 : 8;
  int want = (per_cu * 256 + a.H - 1) / a.H;  // splits per slab
  if (want < 1) want = 1;
  if (want > tiles) want = tiles;
  // Short caches: one split per slab, whose matrix-core kernel writes the output
  // itself.  The first kernel takes 5.4 us for one tile of 256 positions per workgroup
  // and 2 us more for every further one, the merge kernel 3.4 us (8.8 us per call for
  // any S from 512 to 2048 with 32 heads): one more tile costs less than the merge,
  // two cost more (S = 512: 8.8 -> 7.9 us; S = 1024 would be 9.2 -> 11.9).
  if (flash_mfma_applies(a) && a.S <= FL_DIRECT_MAX_S) want = 1;
  const int tiles_per = (tiles + want - 1) / want;
  FlashPlan p;
  p.split_len = tiles_per * FL_TILE;
  p.nsplit = (a.S + p.split_len - 1) / p.split_len;
  return p;
}

size_t flash_scratch_floats(const FlashArgs& a) {
  const FlashPlan p = flash_plan(a);
  return (size_t)a.H * a.group * p.nsplit * (a.D + 2);
}

template <int KIND, int E, int GQ, bool FASTLD>
static hipError_t go(const FlashArgs& a, int qh0, const FlashPlan& pl, float* scratch,
                     hipStream_t s) {
  const int chunks = (a.D + E - 1) / E;
  int LP = 1;
  while (LP < chunks) LP <<= 1;
  const dim3 grid((unsigned)a.H, (unsigned)pl.nsplit);
  if (a.k_out || a.v_out)
    flash_phase1<KIND, E, GQ, true, FASTLD>
        <<<grid, FL_WAVES * 64, 0, s>>>(a, qh0, LP, pl.split_len, scratch);
  else
    flash_phase1<KIND, E, GQ, false, FASTLD>
        <<<grid, FL_WAVES * 64, 0, s>>>(a, qh0, LP, pl.split_len, scratch);
  return hipGetLastError();
}

template <int KIND, int E, bool FASTLD>
static hipError_t go_heads(const FlashArgs& a, const FlashPlan& pl, float* scratch,
                           hipStream_t s) {
  int qh0 = 0;
  while (qh0 < a.group) {
    const int left = a.group - qh0;
    hipError_t e;
    if (left >= 4) {
      e = go<KIND, E, 4, FASTLD>(a, qh0, pl, scratch, s);
      qh0 += 4;
    } else if (left >= 2) {
      e = go<KIND, E, 2, FASTLD>(a, qh0, pl, scratch, s);
      qh0 += 2;
    } else {
      e = go<KIND, E, 1, FASTLD>(a, qh0, pl, scratch, s);
      qh0 += 1;
    }
    if (e != hipSuccess) return e;
  }
  return hipSuccess;
}

hipError_t launch_flash(const FlashArgs& a, float* scratch, hipStream_t s) {
  const FlashPlan pl = flash_plan(a);
  if (pl.nsplit > P2_MAXT) return hipErrorInvalidValue;
  hipError_t e;
  if (try_flash_mfma(a, pl, scratch, s, &e)) {
    if (e != hipSuccess) return e;
    if (pl.nsplit == 1) return hipSuccess;  // that kernel wrote the output
    flash_phase2<<<(unsigned)(a.H * a.group), P2_THREADS, 0, s>>>(scratch, a.out, pl.nsplit, a.D);
    return hipGetLastError();
  }
  const bool al16 = (((uintptr_t)a.k | (uintptr_t)a.v) & 15) == 0;
  if (a.kind == KIND_F16) {
    if (a.D % 8 == 0 && al16) e = go_heads<KIND_F16, 8, true>(a, pl, scratch, s);
    else e = go_heads<KIND_F16, 8, false>(a, pl, scratch, s);
  } else if (a.kind == KIND_W4) {
    if (a.D % 32 == 0 && al16) e = go_heads<KIND_W4, 32, true>(a, pl, scratch, s);
    else e = go_heads<KIND_W4, 8, false>(a, pl, scratch, s);
  } else {
    if (a.D % 16 == 0 && al16) e = go_heads<KIND_F8, 16, true>(a, pl, scratch, s);
    else e = go_heads<KIND_F8, 8, false>(a, pl, scratch, s);
  }
  if (e != hipSuccess) return e;
  flash_phase2<<<(unsigned)(a.H * a.group), P2_THREADS, 0, s>>>(scratch, a.out, pl.nsplit, a.D);
  return hipGetLastError();
}

}  // namespace w4k
