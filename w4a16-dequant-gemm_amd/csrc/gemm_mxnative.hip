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
  // more row tiles per workgroup cut the X traffic, but only pay while several
  // workgroups per CU remain (a second, partly filled round of fat workgroups
  // costs more than it saves)
  const int nt = MT >= 3 ? tiles * mblocks / 512 : 1;
  if (nt >= 3) return launch_decode_nt<MT, 3>(w, x, c, s);
  if (nt >= 2) return launch_decode_nt<MT, 2>(w, x, c, s);
  return launch_decode_nt<MT, 1>(w, x, c, s);
}

}  // namespace

hipError_t launch_gemm_mx_w4a4(const w4_packed_mx_view& w, const w4_packed_mx_view& x,
                               w4_half* c, hipStream_t s) {
  const int M = x.N;
  if (M <= 16) return launch_decode<1>(w, x, c, s);
  if (M <= 32) return launch_decode<2>(w, x, c, s);
  if (M <= 48) return launch_decode<3>(w, x, c, s);
  return launch_decode<4>(w, x, c, s);
}

}  // namespace w4k
