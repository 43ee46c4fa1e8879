// Launch functions of the gfx950 kernels (one per kernel family).  They take
// already-validated arguments and only enqueue work on `stream`.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/w4_abi.h"

namespace w4k {

// Which packed format a weight view carries.
struct WView {
  int mx;  // 0: W4 affine (scales FP16, optional zero-points), 1: MXFP4
  int N, K;
  int gs, G, symmetric;  // W4 only
  int B;                 // MX only
  const uint32_t* q;
  const void* scales;  // w4_half* (W4) or uint8_t* (MX)
  const uint32_t* zeros;
};

inline WView view_of(const w4_packed_view& p) {
  return WView{0, p.N, p.K, p.gs, p.G, p.symmetric, 0, p.q, p.scales, p.zeros};
}
inline WView view_of(const w4_packed_mx_view& p) {
  return WView{1, p.N, p.K, 32, p.B, 1, p.B, p.q, p.scales, nullptr};
}

// dequant.hip
hipError_t launch_dequant(const WView& v, w4_half* w, hipStream_t s);
hipError_t launch_dequant_f8(const uint8_t* q, const w4_half* sc, w4_half* w,
                             int S, int D, int gs, hipStream_t s);

// gemm_simt.hip
hipError_t launch_gemm_simt(const WView& v, const w4_half* x, w4_half* c, int M,
                            hipStream_t s, w4_half* w_out);
// gemm_mfma.hip
hipError_t launch_gemm_mfma(const WView& v, const w4_half* x, w4_half* c, int M,
                            hipStream_t s, w4_half* w_out);

// gemm_tile_dma.hip: large-M W4 kernel with direct-to-LDS operand loads; false
// (nothing launched) when the arguments are not its shape.
bool try_tile_dma(const WView& v, const w4_half* x, w4_half* c, int M, hipStream_t s,
                  w4_half* w_out, hipError_t* err);

// gemm_tile256.hip: the same scheme on 256 x 256 tiles, for try_tile_dma to hand unhooked
// calls to once it has checked the operands; false (nothing launched) when that tile
// would not at least halve the rounds of workgroups on `cus` compute units.
bool try_tile256(const WView& v, const w4_half* x, w4_half* c, int M, hipStream_t s, int cus,
                 hipError_t* err);

// gemm_decode_resident.hip: M <= 64 with the activations fetched once per workgroup
// (several 16-row tiles each).  Same order of additions as the K-split decode
// kernels of gemm_mfma.hip, which serve the hooked calls of these shapes.
bool decode_resident_applies(const WView& v, const w4_half* x, const w4_half* c, int M);
hipError_t launch_decode_resident(const WView& v, const w4_half* x, w4_half* c, int M,
                                  hipStream_t s);
// Long K (8, 11 or 14 chunks of 128 k per wave) with more than 12 to 16 activation rows on a grid of
// more tiles than compute units: the resident kernel then gives a workgroup two tiles, and the
// long-K kernel below leaves the shape to it.
bool decode_resident_shares_long_k(const WView& v, const w4_half* x, const w4_half* c, int M);

// gemm_decode_longk.hip: M <= 64 at long K (5 to 16 chunks of 128 k per wave; 2 to 4 on thin grids), one
// 16-row tile per workgroup with activations and codes requested chunk by chunk while
// earlier chunks multiply; same order of additions as the two kernels above.
bool decode_longk_applies(const WView& v, const w4_half* x, const w4_half* c, int M);
hipError_t launch_decode_longk(const WView& v, const w4_half* x, w4_half* c, int M,
                               hipStream_t s);

// gemm_decode_general.hip: M <= 64 for any group size (multiple of 8) and any K % 8 == 0
// with 1024 < K <= 5120, group parameters through LDS; same order of additions as the
// K-split decode kernels of gemm_mfma.hip.
bool decode_general_applies(const WView& v, const w4_half* x, const w4_half* c, int M);
hipError_t launch_decode_general(const WView& v, const w4_half* x, w4_half* c, int M,
                                 hipStream_t s);

// flash.hip -- one description for the four cache kinds
struct FlashArgs {
  int kind;  // 0 FP16, 1 W4, 2 FP8
  int H;     // cache slabs addressed by a (sequence, kv-head) pair: nseq * Hkv
  int S, D, gs, G, symmetric;
  int group;       // query heads per slab
  int scale_mode;  // FP8: 0 per (row, group), 1 per slab
  const void* k;   // FP16: halves; W4: packed words; FP8: bytes
  const void* v;
  const w4_half* s_k;
  const w4_half* s_v;
  const uint32_t* z_k;
  const uint32_t* z_v;
  // paging (W4 only): bt == nullptr means contiguous slabs of S rows
  const int* bt;
  int bt_stride;   // entries per sequence table
  int page, pool_rows;
  int Hkv;         // paged: pool slabs; sequence = slab / Hkv
  const w4_half* q;
  w4_half* out;
  w4_half* k_out;
  w4_half* v_out;
};
enum { KIND_F16 = 0, KIND_W4 = 1, KIND_F8 = 2 };  // FlashArgs::kind

// Split of the sequence over workgroups (shared by both phase-1 kernels).
constexpr int FL_DIRECT_MAX_S = 512;  // longest cache served by one split per slab
struct FlashPlan {
  int split_len, nsplit;
};
FlashPlan flash_plan(const FlashArgs& a);
// flash_mfma.hip: whether the matrix-core phase 1 (D = 128) takes these arguments.
bool flash_mfma_applies(const FlashArgs& a);
// Launches it; false when the arguments need the general kernel (nothing is
// launched then).
bool try_flash_mfma(const FlashArgs& a, const FlashPlan& pl, float* part, hipStream_t s,
                    hipError_t* err);

// Floats of scratch the split-S partials need for these arguments.
size_t flash_scratch_floats(const FlashArgs& a);
hipError_t launch_flash(const FlashArgs& a, float* scratch, hipStream_t s);

// quantize.hip -- the host quantizers as kernels.  mode: 0 W4 symmetric, 1 W4 with
// zero-points, 2 E4M3 bytes; src is FP64 or (src_f16) FP16; `rows` rows of K
// elements, groups of gs along K.  status: bit 0 non-finite input, bit 1 scale
// out of range (OR-ed in by the kernels).
struct QuantSide {  // one source and its outputs (q32: W4 words, q8: E4M3 bytes)
  const void* src;
  uint32_t* q32;
  uint8_t* q8;
  w4_half* scales;
  uint32_t* zeros;
};
// nsides (1 or 2) jobs of the same shape in one launch: the K and V sides of a cache
hipError_t launch_quantize_rows(int mode, const QuantSide* sides, int nsides, int src_f16,
                                long long rows, int K, int gs, int* status, hipStream_t s);
hipError_t launch_quantize_mx(const void* src, int src_f16, long long rows, int K, uint32_t* q,
                              uint8_t* scales, int* status, hipStream_t s);
// gemm_mxnative.hip -- both operands packed MXFP4 (x.N = M rows of K), scaled MFMA
hipError_t launch_gemm_mx_w4a4(const w4_packed_mx_view& w, const w4_packed_mx_view& x,
                               w4_half* c, hipStream_t s);
hipError_t launch_gemm_mx_w4a8(const w4_packed_mx_view& w, const w4_act_mx8_view& x, w4_half* c,
                               hipStream_t s);
hipError_t launch_quantize_mx8(const void* src, int src_f16, long long rows, int K, uint8_t* q,
                               uint8_t* scales, int* status, hipStream_t s);
hipError_t launch_fill_words(uint32_t* p, long long n, uint32_t value, hipStream_t s);

}  // namespace w4k
