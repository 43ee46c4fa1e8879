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

// One MFMA over the 32-blocks picked by SEL: byte SEL of each lane's scale word.
template <int SEL>
__device__ __forceinline__ f4 mfma_fp4(u4 a, uint32_t sa, u4 b, uint32_t sb, f4 c) {
  const v4i a4 = __builtin_bit_cast(v4i, a), b4 = __builtin_bit_cast(v4i, b);
  // FP4 operands occupy the low four of the eight operand registers
  const v8i va = __builtin_shufflevector(a4, a4, 0, 1, 2, 3, -1, -1, -1, -1);
  const v8i vb = __builtin_shufflevector(b4, b4, 0, 1, 2, 3, -1, -1, -1, -1);
  return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(va, vb, c, FMT_FP4, FMT_FP4, SEL,
                                                          (int)sa, SEL, (int)sb);
}

// The four consecutive 32-blocks b0..b0+3 of one packed row (64 bytes of codes)
// and their four scale bytes as one word.  FULL: every block exists and rows
// are 16-byte aligned.  Otherwise words past the row read as zero codes, codes
// past K are masked off, and missing blocks take the neutral scale byte 127.
template <bool FULL>
__device__ __forceinline__ void load_blocks(const uint32_t* __restrict__ qrow,
                                            const uint8_t* __restrict__ srow, int b0, int B,
                                            int wk, int K, u4 q[4], uint32_t& sc) {
  if (FULL) {
#pragma unroll
    for (int j = 0; j < 4; ++j) q[j] = *(const u4*)(qrow + (size_t)(b0 + j) * 4);
    sc = *(const uint32_t*)(srow + b0);
  } else {
    sc = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int b = b0 + j;
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const int wi = b * 4 + t;
        uint32_t word = wi < wk ? qrow[wi] : 0u;
        if (wi == wk - 1 && (K & 7)) word &= (1u << (4 * (K & 7))) - 1u;
        q[j][t] = word;
      }
      sc |= (uint32_t)(b < B ? srow[b] : (uint8_t)127) << (8 * j);
    }
  }
}

// Skinny M: a workgroup owns 16 rows of W and 16*MT rows of X (grid.y walks
// further X rows); its 8 waves take 512-k super-steps round-robin.  Inside a
// super-step lane group g = l/16 holds blocks 4g..4g+3 of its row, and MFMA j
// contracts block 4g+j of every group: the k order inside a super-step is
// permuted identically for both operands.  Partial sums meet in LDS and are
// added in wave order.
template <int MT, bool FULL>
__global__ __launch_bounds__(NV_WAVES * 64) void mxn_decode_kernel(
    const uint32_t* __restrict__ wq, const uint8_t* __restrict__ ws,
    const uint32_t* __restrict__ xq, const uint8_t* __restrict__ xs, w4_half* __restrict__ c,
    int N, int K, int B, int M) {
  __shared__ f4 red[NV_WAVES][MT][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int wk = words(K);
  const int n0 = blockIdx.x * 16, m0 = blockIdx.y * (16 * MT);
  const int n = n0 + r < N ? n0 + r : N - 1;
  const uint32_t* wrow = wq + (size_t)n * wk;
  const uint8_t* wsrow = ws + (size_t)n * B;
  const uint32_t* xrow[MT];
  const uint8_t* xsrow[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = m0 + mt * 16 + r < M ? m0 + mt * 16 + r : M - 1;
    xrow[mt] = xq + (size_t)m * wk;
    xsrow[mt] = xs + (size_t)m * B;
  }
  f4 acc[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) acc[mt] = f4{0.f, 0.f, 0.f, 0.f};

  const int supers = (B + 15) >> 4;
  for (int ss = wave; ss < supers; ss += NV_WAVES) {
    const int b0 = ss * 16 + g * 4;
    u4 a[4];
    uint32_t sa;
    load_blocks<FULL>(wrow, wsrow, b0, B, wk, K, a, sa);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      u4 b[4];
      uint32_t sb;
      load_blocks<FULL>(xrow[mt], xsrow[mt], b0, B, wk, K, b, sb);
      acc[mt] = mfma_fp4<0>(a[0], sa, b[0], sb, acc[mt]);
      acc[mt] = mfma_fp4<1>(a[1], sa, b[1], sb, acc[mt]);
      acc[mt] = mfma_fp4<2>(a[2], sa, b[2], sb, acc[mt]);
      acc[mt] = mfma_fp4<3>(a[3], sa, b[3], sb, acc[mt]);
    }
  }
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) red[wave][mt][lane] = acc[mt];
  __syncthreads();
  // MT * 64 lane slots of four n each
  for (int o = threadIdx.x; o < MT * 64; o += NV_WAVES * 64) {
    const int mt = o >> 6, l = o & 63;
    f4 sum = red[0][mt][l];
#pragma unroll
    for (int w = 1; w < NV_WAVES; ++w) sum += red[w][mt][l];
    const int m = m0 + mt * 16 + (l & 15), nn = n0 + 4 * (l >> 4);
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

template <int MT>
hipError_t launch_decode(const w4_packed_mx_view& w, const w4_packed_mx_view& x, w4_half* c,
                         hipStream_t s) {
  const int N = w.N, K = w.K, M = x.N;
  const bool full = K % 512 == 0 && ((uintptr_t)w.q & 15) == 0 && ((uintptr_t)x.q & 15) == 0 &&
                    ((uintptr_t)w.scales & 3) == 0 && ((uintptr_t)x.scales & 3) == 0;
  const dim3 grid((unsigned)((N + 15) / 16), (unsigned)((M + 16 * MT - 1) / (16 * MT)));
  const dim3 block(NV_WAVES * 64);
  if (full)
    mxn_decode_kernel<MT, true><<<grid, block, 0, s>>>(w.q, w.scales, x.q, x.scales, c, N, K,
                                                      w.B, M);
  else
    mxn_decode_kernel<MT, false><<<grid, block, 0, s>>>(w.q, w.scales, x.q, x.scales, c, N, K,
                                                       w.B, M);
  return hipGetLastError();
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
