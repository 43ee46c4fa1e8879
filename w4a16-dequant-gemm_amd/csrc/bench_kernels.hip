// Bandwidth yardsticks for the benchmark (not part of the C ABI the tests
// bind): a streaming read that folds every dwordx4 into a register, and a
// dwordx4 copy.  The measured rates are the denominators the fused kernels'
// achieved GB/s are compared with, next to the 8 TB/s HBM3E figure.
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef uint32_t u4 __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(256) void stream_read(const u4* __restrict__ src, size_t n16,
                                                   uint32_t* __restrict__ sink) {
  size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * 256;
  u4 acc = {0u, 0u, 0u, 0u};
  for (; i + 3 * stride < n16; i += 4 * stride) {
    const u4 a = __builtin_nontemporal_load(src + i);
    const u4 b = __builtin_nontemporal_load(src + i + stride);
    const u4 c = __builtin_nontemporal_load(src + i + 2 * stride);
    const u4 d = __builtin_nontemporal_load(src + i + 3 * stride);
    acc ^= a ^ b ^ c ^ d;
  }
  for (; i < n16; i += stride) acc ^= __builtin_nontemporal_load(src + i);
  const uint32_t r = acc[0] ^ acc[1] ^ acc[2] ^ acc[3];
  if (r == 0x9E3779B9u) sink[0] = r;  // practically never; keeps the loads alive
}

__global__ __launch_bounds__(256) void stream_copy(const u4* __restrict__ src,
                                                   u4* __restrict__ dst, size_t n16) {
  size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * 256;
  for (; i < n16; i += stride) __builtin_nontemporal_store(__builtin_nontemporal_load(src + i), dst + i);
}

extern "C" int w4bench_read(const void* src, size_t bytes, void* sink, int blocks, void* stream) {
  stream_read<<<blocks, 256, 0, (hipStream_t)stream>>>((const u4*)src, bytes / 16, (uint32_t*)sink);
  return (int)hipGetLastError();
}

extern "C" int w4bench_copy(const void* src, void* dst, size_t bytes, int blocks, void* stream) {
  stream_copy<<<blocks, 256, 0, (hipStream_t)stream>>>((const u4*)src, (u4*)dst, bytes / 16);
  return (int)hipGetLastError();
}

// Host-side launch loop: `steps` back-to-back calls of one GEMM entry point,
// rotating through `nviews` weight views, without returning to the caller's
// interpreter between launches.
typedef int (*w4bench_gemm_fn)(const void* view, const void* x, void* c, int M, void* stream,
                               void* w_out);
extern "C" int w4bench_gemm_loop(w4bench_gemm_fn fn, const void* const* views, int nviews,
                                 const void* x, void* c, int M, int steps, void* stream) {
  for (int i = 0; i < steps; ++i) {
    const int rc = fn(views[i % nviews], x, c, M, stream, nullptr);
    if (rc) return rc;
  }
  return 0;
}

// The same loop for the two-view W4A4 / W4A8 entry points.
typedef int (*w4bench_w4a4_fn)(const void* w_view, const void* x_view, void* c, void* stream);
extern "C" int w4bench_w4a4_loop(w4bench_w4a4_fn fn, const void* const* views, int nviews,
                                 const void* x_view, void* c, int steps, void* stream) {
  for (int i = 0; i < steps; ++i) {
    const int rc = fn(views[i % nviews], x_view, c, stream);
    if (rc) return rc;
  }
  return 0;
}
