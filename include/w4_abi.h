/*
 * C ABI of libw4amd.so: the gfx950 launcher behind the w4::gpu C++ API.
 *
 * Every entry point validates its arguments before it touches the device (a
 * bad call never dereferences a pointer, allocates or launches), then enqueues
 * its kernels on `stream` and returns without synchronising.  All data
 * pointers are device pointers owned by the caller.  Halves cross the boundary
 * as IEEE binary16 bit patterns (w4_half has the storage of __half).
 *
 * Return value: W4_OK, W4_EINVAL (the reference throws std::invalid_argument
 * here) or W4_ERUNTIME (the reference throws std::runtime_error from
 * cuda_check).  w4_last_error() returns the thread's last message.
 *
 * The citations name the reference function each entry point replaces
 * (paths relative to the reference repository).
 */
#ifndef W4_ABI_H
#define W4_ABI_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef uint16_t w4_half;
typedef void* w4_stream; /* hipStream_t; NULL is the default stream */

enum { W4_OK = 0, W4_EINVAL = 1, W4_ERUNTIME = 2 };

/* Packed W4 weights, device view.  include/w4/dequant.cuh:31-37 */
typedef struct w4_packed_view {
  int N, K, gs, G;
  int symmetric;
  const uint32_t* q;     /* N * words(K), 8 nibbles per word, low first   */
  const w4_half* scales; /* N * G                                          */
  const uint32_t* zeros; /* N * words(G) nibbles; NULL when symmetric      */
} w4_packed_view;

/* Packed MXFP4 weights, device view.  include/w4/mxfused.cuh:26-30 */
typedef struct w4_packed_mx_view {
  int N, K, B;           /* B = ceil(K / 32)                               */
  const uint32_t* q;     /* N * words(K) E2M1 codes                        */
  const uint8_t* scales; /* N * B E8M0 bytes                               */
} w4_packed_mx_view;

/* W4 KV cache, device view: H slabs of S rows.  include/w4/kvattention.cuh:39-48 */
typedef struct w4_kv_view {
  int H, S, D, gs, G;
  int symmetric;
  const uint32_t* q_k;
  const w4_half* s_k;
  const uint32_t* z_k;
  const uint32_t* q_v;
  const w4_half* s_v;
  const uint32_t* z_v;
} w4_kv_view;

/* FP8-E4M3 KV cache, device view.  include/w4/kvflash.cuh:390-396 */
typedef struct w4_kv_f8_view {
  int H, S, D, gs, G;
  const uint8_t* q_k;
  const w4_half* s_k;
  const uint8_t* q_v;
  const w4_half* s_v;
} w4_kv_f8_view;

/* MXFP8 activations, device view: E4M3 bytes under one E8M0 scale per 32 along K
 * (no counterpart in the reference; host side: include/w4/mxact.hpp here). */
typedef struct w4_act_mx8_view {
  int M, K, B;           /* B = ceil(K / 32)                               */
  const uint8_t* q;      /* M * K E4M3 bytes                               */
  const uint8_t* scales; /* M * B E8M0 bytes                               */
} w4_act_mx8_view;

const char* w4_last_error(void);

/* M at or above this goes to the matrix-core kernel in w4_gemm / w4_gemm_mx.
 * include/w4/dispatch.cuh:25 (re-measured for gfx950). */
int w4_dispatch_mma_min_m(void);
/* The same for one weight matrix: rows of packed words that are not 16-byte aligned
 * (K % 32 != 0) leave the vector kernels their word-by-word form, and on large matrices
 * (N * K >= 2^25) the matrix-core kernel is ahead from M = 2 (N = 11008, K = 4104: M = 2 / 4
 * 19.2 / 32.6 us against 18.5).  So it is for K above 4096 (K % 32 == 0; W4 and MXFP4):
 * three or four activation rows cost the vector kernels a second pass over their
 * staged activations, the matrix-core kernel fetches only the rows that exist
 * (N = 4096, K = 11008, M = 3: 18.2 us against 9.0; up to K = 6144 in whole chunks of
 * 128 already from M = 2), and for wide matrices at K <= 4096 (N * K >= 172 000 per compute unit,
 * 44 M on an MI355X: N = 11008 or
 * 14336 at K = 4096, M = 3 / 4: 8.6 - 9.6 us against 9.4 - 11.8).  Everywhere else this is
 * w4_dispatch_mma_min_m().  No counterpart in the reference, whose crossover is one
 * constant (dispatch.cuh:25). */
int w4_dispatch_mma_min_m_for(int N, int K);
/* What w4_gemm uses: the same with the group size taken into account (a group size that is
 * no multiple of 32 keeps w4_dispatch_mma_min_m() on wide matrices at K <= 4096: its
 * matrix-core kernel looks group parameters up per packed word and is behind the vector
 * kernel through M = 4; gs <= 0 means "a multiple of 32").  No counterpart in the reference. */
int w4_dispatch_mma_min_m_for_gs(int N, int K, int gs);
/* The same for an MXFP4 matrix (what w4_gemm_mx uses): as above, and 2 for K above 4096 other
 * than 8192 (N = 4096, K = 14336, M = 2: 9.8 us against 11.5).  No counterpart in the reference. */
int w4_dispatch_mma_min_m_for_mx(int N, int K);

/* ---- packed-weight GEMM: c[M,N] = x[M,K] * W[N,K]^T, FP16 in/out ---------- */
/* w: N*K halves, bit-identical to the host dequant_all.  dequant.cuh:62-82 */
int w4_dequant(const w4_packed_view* p, w4_half* w, w4_stream stream);
/* fused.cuh:172-214; w_out (optional) receives every dequantized weight */
int w4_gemm_fused(const w4_packed_view* p, const w4_half* x, w4_half* c, int M,
                  w4_stream stream, w4_half* w_out);
/* mma.cuh:234-260 */
int w4_gemm_mma(const w4_packed_view* p, const w4_half* x, w4_half* c, int M,
                w4_stream stream, w4_half* w_out);
/* dispatch.cuh:27-34 */
int w4_gemm(const w4_packed_view* p, const w4_half* x, w4_half* c, int M,
            w4_stream stream, w4_half* w_out);

/* mxfused.cuh:57-69, 166-198, 291-307; dispatch.cuh:36-43 */
int w4_dequant_mx(const w4_packed_mx_view* p, w4_half* w, w4_stream stream);
int w4_gemm_fused_mx(const w4_packed_mx_view* p, const w4_half* x, w4_half* c,
                     int M, w4_stream stream, w4_half* w_out);
int w4_gemm_mma_mx(const w4_packed_mx_view* p, const w4_half* x, w4_half* c,
                   int M, w4_stream stream, w4_half* w_out);
int w4_gemm_mx(const w4_packed_mx_view* p, const w4_half* x, w4_half* c, int M,
               w4_stream stream, w4_half* w_out);

/* Plain FP16 GEMM (FP32 accumulate) over already-dequantized W: the two-pass
 * baseline.  dequant.cuh:87-100 (cublasGemmEx there, hipBLASLt here). */
int w4_gemm_fp16(const w4_half* w, const w4_half* x, w4_half* c, int M, int N,
                 int K, w4_stream stream);

/* ---- split-S flash-decode attention: one query token per head ------------- */
/* kvflash.cuh:350-363.  q, out: H*D halves; k_out/v_out (optional): H*S*D */
int w4_attention_w4_flash(const w4_kv_view* p, const w4_half* q, w4_half* out,
                          w4_stream stream, w4_half* k_out, w4_half* v_out);
/* kvflash.cuh:365-384 */
int w4_attention_fp16_flash(const w4_half* q, const w4_half* k16,
                            const w4_half* v16, w4_half* out, int H, int S,
                            int D, w4_stream stream);
/* kvflash.cuh:572-590 */
int w4_attention_f8_flash(const w4_kv_f8_view* p, const w4_half* q,
                          w4_half* out, w4_stream stream, w4_half* k_out,
                          w4_half* v_out);
/* kvflash.cuh:725-764.  p->S is the logical length; each head's pool slab has
 * npages*page rows; logical row t lives at bt[t/page]*page + t%page. */
int w4_attention_w4_flash_paged(const w4_kv_view* p, const int* bt, int page,
                                int npages, const w4_half* q, w4_half* out,
                                w4_stream stream, w4_half* k_out,
                                w4_half* v_out);
/* kvflash.cuh:435-457: rows of E4M3 bytes -> halves, scale per (row, group) */
int w4_dequant_f8(const uint8_t* q, const w4_half* s, w4_half* w, int S, int D,
                  int gs, w4_stream stream);

/* ---- batched / grouped-query forms (no counterpart in the reference, which
 * has one query head per cache slab and one block table per call).  The cache
 * views hold B*Hkv slabs; `group` = Hq/Hkv query heads share each slab, so q
 * and out are (H*group)*D halves ordered slab-major.  group = 1 reduces to the
 * entry points above. ------------------------------------------------------- */
int w4_attention_w4_flash_gqa(const w4_kv_view* p, int group, const w4_half* q,
                              w4_half* out, w4_stream stream, w4_half* k_out,
                              w4_half* v_out);
int w4_attention_fp16_flash_gqa(const w4_half* q, const w4_half* k16,
                                const w4_half* v16, w4_half* out, int H,
                                int group, int S, int D, w4_stream stream);
/* scale_mode 0: s_k/s_v hold one FP16 scale per (row, group) as in the
 * reference; 1: one FP16 scale per slab (s_k/s_v have p->H entries). */
int w4_attention_f8_flash_gqa(const w4_kv_f8_view* p, int group, int scale_mode,
                              const w4_half* q, w4_half* out, w4_stream stream,
                              w4_half* k_out, w4_half* v_out);
/* One pool shared by all sequences: the view's H = Hkv slabs of npages*page
 * rows; bt holds nseq tables of bt_stride entries; sequence s reads slab
 * (s, h) -> pool slab h through table s.  q/out: nseq*Hkv*group*D halves. */
int w4_attention_w4_flash_paged_batched(const w4_kv_view* p, const int* bt,
                                        int nseq, int bt_stride, int page,
                                        int npages, int group,
                                        const w4_half* q, w4_half* out,
                                        w4_stream stream);

/* No counterpart in the reference: w4_attention_w4_flash_gqa for callers that
 * cannot allocate device memory (HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc).  Same arguments, kernels and output bytes;
 * the split-S partials live in a W4_NOALLOC_SCRATCH_BYTES array built into the
 * library (one copy per GPU, held until the process ends) instead of the
 * library's grow-only buffer, and the call makes no hipMalloc / hipFree.  Calls
 * whose partials (slabs * group * splits * (D + 2) floats, splits chosen so that
 * about 512 workgroups run) do not fit are rejected with W4_EINVAL.  Every call
 * on one GPU shares that GPU's array: calls that overlap on one GPU race. */
#define W4_NOALLOC_SCRATCH_BYTES (4u << 20)
int w4_attention_w4_flash_gqa_noalloc(const w4_kv_view* p, int group,
                                      const w4_half* q, w4_half* out,
                                      w4_stream stream, w4_half* k_out,
                                      w4_half* v_out);

/* ---- device-side quantizers: the host quantizers as kernels, same bytes -----
 * The view's arrays are the OUTPUTS (device memory of the sizes the view
 * implies; no need to clear them).  Sources are row-major FP64, as the host
 * quantizers take them; the cache forms also take FP16 sources (src_f16 != 0),
 * which quantize as the same values widened to FP64.  What the host reports by
 * throwing after looking at the data lands in *status (a device int, cleared
 * by the call): bit 0 non-finite input, bit 1 a group scale outside the FP16
 * (E8M0 for MXFP4) range (non-finite input may set both; the host reports it
 * first).  Outputs are unspecified when it ends non-zero. */
/* include/w4/pack.hpp:64-130 */
int w4_quantize(const w4_packed_view* out, const double* w, int* status,
                w4_stream stream);
/* include/w4/mx.hpp:71-119 */
int w4_quantize_mx(const w4_packed_mx_view* out, const double* w, int* status,
                   w4_stream stream);
/* the same quantizer over FP16 sources (activations): out->N rows of out->K */
int w4_quantize_mx_f16(const w4_packed_mx_view* out, const w4_half* x,
                       int* status, w4_stream stream);
/* include/w4/kvcache.hpp:60-108; k, v: H*S*D elements, head- then row-major */
int w4_quantize_cache(const w4_kv_view* out, const void* k, const void* v,
                      int src_f16, int* status, w4_stream stream);
/* include/w4/kvfp8.hpp:70-128 */
int w4_quantize_cache_f8(const w4_kv_f8_view* out, const void* k, const void* v,
                         int src_f16, int* status, w4_stream stream);

/* ---- W4A4 on the scaled matrix cores (no counterpart in the reference, whose
 * MXFP4 kernels keep FP16 activations: include/w4/mxfused.cuh:166-198,291-307).
 * c[M,N] = X[M,K] * W[N,K]^T with both operands packed MXFP4 (x->N = M rows,
 * x->K == w->K).  E2M1 products and E8M0 scales are exact; accumulation is
 * FP32, the output FP16.  Its gate is separate from the W4A16 one: rel L2
 * <= 1e-3 against the FP64 product of the two dequantized operands.  Codes
 * past K in a row's last word are ignored. */
int w4_gemm_mx_w4a4(const w4_packed_mx_view* w, const w4_packed_mx_view* x,
                    w4_half* c, w4_stream stream);

/* W4A8: MXFP4 weights against MXFP8 activations (E4M3 elements, E8M0 block
 * scales; w4_quantize_mx8_f16 makes them from FP16 with the bytes of the host
 * mxa::quantize_mx8).  Same exactness and gate as W4A4.  K must be a multiple
 * of 32 and x->q 16-byte aligned. */
int w4_quantize_mx8_f16(const w4_act_mx8_view* out, const w4_half* x, int* status,
                        w4_stream stream);
int w4_gemm_mx_w4a8(const w4_packed_mx_view* w, const w4_act_mx8_view* x,
                    w4_half* c, w4_stream stream);

#ifdef __cplusplus
}
#endif
#endif
