/*
 * CPU oracle for the fused-dequant hot path -- TEST INFRASTRUCTURE ONLY.
 *
 * A plain-C restatement of the reference's host arithmetic (packed W4 / MXFP4
 * weights, W4 / FP8 / paged KV caches, FP64 GEMM and attention references).
 * It exists to check the HIP kernels and the C++ host headers; nothing that
 * ships may call it.  Only tests, the smoke check and the CPU-baseline leg of
 * the benchmark load this library.
 *
 * Halves are carried as raw IEEE binary16 bit patterns (uint16_t) and converted
 * in software, so the file builds with plain gcc and shares no code with the
 * HIP half type the product uses.
 *
 * Every function returns 0 on success and ORC_EINVAL where the reference
 * throws std::invalid_argument; orc_last_error() gives the message.
 *
 * Parity status: every function below is pinned by at least one
 * reference-held known answer or mathematical invariant in tests/ (see the
 * per-function notes in w4_oracle.c).
 */
#ifndef W4_ORACLE_H
#define W4_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ORC_OK 0
#define ORC_EINVAL 1

const char* orc_last_error(void);

/* ---- scalar steps ------------------------------------------------------ */
uint16_t orc_f32_to_f16(float f);           /* round-to-nearest-even        */
float orc_f16_to_f32(uint16_t h);
uint16_t orc_dequant_one(uint16_t s, int q, int z);       /* pack.hpp:58-60  */
uint16_t orc_dequant_one_mx(uint8_t se, int q);           /* mx.hpp:56-63    */
float orc_decode_f8_e4m3(uint8_t b);                      /* kvfp8.hpp:42-47 */
uint16_t orc_dequant_one_f8(uint16_t s, uint8_t b);       /* kvfp8.hpp:51-53 */
uint8_t orc_f32_to_e4m3_satfinite(float x);  /* RNE, OCP E4M3, clamp +-448   */

/* ---- seeded generators (pack.hpp:186-200; libstdc++ streams) ------------ */
void orc_mt19937_64_stream(uint64_t seed, uint64_t* out, size_t n);
void orc_normal_weights(double* out, size_t n, uint64_t seed);
void orc_normal_activations(uint16_t* out, size_t n, uint64_t seed);
/* error_analysis.cpp:44-61,134-137 (only to reproduce its recorded tables) */
void orc_laplace_weights(double* out, size_t n, uint64_t seed);
void orc_uniform_weights(double* out, size_t n, uint64_t seed);
void orc_uniform_int_stream(uint64_t seed, uint64_t range, uint64_t* out,
                            size_t n);

/* ---- W4 (pack.hpp) ------------------------------------------------------ */
int orc_words(int n);
int orc_quantize(const double* w, size_t w_len, int N, int K, int gs,
                 int symmetric, uint32_t* q, uint16_t* scales,
                 uint32_t* zeros);
int orc_dequant_all(int N, int K, int gs, int G, int symmetric,
                    const uint32_t* q, size_t q_len, const uint16_t* scales,
                    size_t s_len, const uint32_t* zeros, size_t z_len,
                    uint16_t* w);
int orc_gemm_oracle(const uint16_t* x, size_t x_len, int M, int K,
                    const uint16_t* w, size_t w_len, int N, double* c);

/* ---- MXFP4 (mx.hpp) ----------------------------------------------------- */
int orc_blocks(int K);
int orc_quantize_mx(const double* w, size_t w_len, int N, int K, uint32_t* q,
                    uint8_t* scales);
int orc_dequant_all_mx(int N, int K, int B, const uint32_t* q, size_t q_len,
                       const uint8_t* scales, size_t s_len, uint16_t* w);

/* ---- W4 KV cache (kvcache.hpp) ------------------------------------------ */
int orc_quantize_cache(const double* k, size_t k_len, const double* v,
                       size_t v_len, int H, int S, int D, int gs,
                       int symmetric, uint32_t* q_k, uint16_t* s_k,
                       uint32_t* z_k, uint32_t* q_v, uint16_t* s_v,
                       uint32_t* z_v);
/* softmax(q K^T / sqrt(D)) V in FP64 over FP16-exact K/V, one query per head.
 * k16/v16 are H slabs of S*D halves; `heads_per_slab` query heads share each
 * slab (1 = the reference's layout; >1 = grouped-query attention).  q is
 * (H*heads_per_slab)*D halves, out the same count of doubles.
 * Follows kvcache.hpp:141-175 once the cache is dequantized. */
int orc_attention_f16(const uint16_t* q, const uint16_t* k16,
                      const uint16_t* v16, int H, int heads_per_slab, int S,
                      int D, double* out);

/* ---- FP8 KV cache (kvfp8.hpp) ------------------------------------------- */
int orc_quantize_cache_f8(const double* k, size_t k_len, const double* v,
                          size_t v_len, int H, int S, int D, int gs,
                          uint8_t* q_k, uint16_t* s_k, uint8_t* q_v,
                          uint16_t* s_v);
int orc_dequant_f8(const uint8_t* q, const uint16_t* s, int rows, int D,
                   int gs, uint16_t* w);

/* ---- paged W4 KV cache (kvpaged.hpp:72-134) ------------------------------ */
/* Scatter `rows_per_head`=S logical rows of `row_elems` elements (elem_size
 * bytes each) per head into a pool of npages*page rows per head. */
int orc_paged_scatter(const void* src, void* dst, int H, int S, int page,
                      const int* bt, int bt_len, size_t row_elems,
                      size_t elem_size);

/* ---- MXFP8 activations (additive: the reference has no such format) --------
 * E4M3 elements under one E8M0 scale per 32, defined by analogy with
 * mx.hpp:71-119: the block exponent is the smallest e with amax <= 448 * 2^e
 * (clamped to [-127, 127]; larger fails), an element is the RNE / saturating
 * E4M3 code (kvfp8.hpp:48-53) of float(v / 2^e).  Pinned by closed forms in the
 * CPU suite (exact round trip of representable values, block maxima on both
 * sides of 448 * 2^e, agreement with the independent C++ header). */
int orc_quantize_mx8(const double* x, size_t x_len, int M, int K, uint8_t* q,
                     uint8_t* scales);
int orc_dequant_mx8(int M, int K, const uint8_t* q, const uint8_t* scales,
                    double* out);
/* c[m][n] = sum_k x[m][k] * w[n][k] over FP64 operands (pack.hpp:150-170
 * without the FP16 widening). */
int orc_gemm_f64(const double* x, int M, int K, const double* w, int N, double* c);

/* ---- helpers ------------------------------------------------------------- */
/* sqrt(sum((half(b)-a)^2)/sum(a^2)): the benches' quantization-error figure. */
double orc_rel_l2_f16_vs_f64(const double* a, const uint16_t* b, size_t n);
double orc_max_abs_f16_vs_f64(const double* a, const uint16_t* b, size_t n);
void orc_set_threads(int n); /* rows of the FP64 references run in parallel */

#ifdef __cplusplus
}
#endif
#endif
