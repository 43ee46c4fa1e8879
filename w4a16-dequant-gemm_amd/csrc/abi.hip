// The C ABI of libw4amd.so: argument contracts first, then launches.
//
// Each entry point rejects a malformed call before any device work: the checks
// read only the view structs and compare pointers with null, so a bad call
// never dereferences, allocates or launches.  The contract lists follow the
// reference launch wrappers (dequant.cuh:63-77, fused.cuh:175-194,
// mma.cuh:237-254, mxfused.cuh:32-37,59-64,169-178,294-301,
// kvflash.cuh:37-54,368-376,437-452,579-582,733-754).
#include <hip/hip_runtime.h>
#include <limits.h>
#include <stdio.h>

#include <atomic>
#include <mutex>

#include "kernels.h"

namespace {

thread_local char g_msg[256] = "";

int invalid(const char* msg) {
  snprintf(g_msg, sizeof g_msg, "%s", msg);
  return W4_EINVAL;
}

int runtime(const char* what, hipError_t e) {
  snprintf(g_msg, sizeof g_msg, "%s: %s", what, hipGetErrorString(e));
  return W4_ERUNTIME;
}

#define REQUIRE(cond, msg) \
  do {                     \
    if (!(cond)) return invalid(msg); \
  } while (0)

int done(const char* what, hipError_t e) {
  return e == hipSuccess ? W4_OK : runtime(what, e);
}

// Measured on MI355X (N = 4096 and 11008, K = 4096, gs = 128): the vector kernel
// wins through M = 4 (5.8 vs 6.2 us and 12.7 vs 13.9 us at M = 4) and loses from
// M = 5 on, where it needs a second pass over the activations (11.8 vs 6.5 us and
// 34 vs 16 us at M = 8).
constexpr int DISPATCH_MMA_MIN_M = 5;

// Largest M the reference's launch grids accept; kept so callers see the same
// rejections (fused.cuh:187-194, mma.cuh:253-254).
constexpr long long FUSED_MAX_M = 65535LL * 4;
constexpr long long MMA_MAX_M = 65535LL * 64;

int check_packed(const w4_packed_view* p, const char* who) {
  static thread_local char buf[96];
#define PK(cond, text)                                   \
  do {                                                   \
    if (!(cond)) {                                       \
      snprintf(buf, sizeof buf, "%s: %s", who, text);    \
      return invalid(buf);                               \
    }                                                    \
  } while (0)
  PK(p != nullptr, "null view");
  PK(p->N >= 1 && p->K >= 1, "bad dims");
  PK(p->gs >= 8 && p->gs % 8 == 0, "gs must be a multiple of 8");
  PK(p->G == (p->K + p->gs - 1) / p->gs, "G inconsistent with K, gs");
  PK(p->q && p->scales, "null pointer");
  PK(p->symmetric || p->zeros, "asymmetric without zeros");
  PK(!p->symmetric || !p->zeros, "symmetric carries no zeros");
#undef PK
  return W4_OK;
}

int check_mx(const w4_packed_mx_view* p) {
  REQUIRE(p != nullptr, "mx: null view");
  REQUIRE(p->N >= 1 && p->K >= 1, "mx: bad dims");
  REQUIRE(p->B == (p->K + 31) / 32, "mx: B inconsistent with K");
  REQUIRE(p->q && p->scales, "mx: null pointer");
  return W4_OK;
}

// Grow-only device scratch for the split-S partials, one per device, shared by all
// calls on that device (calls on different streams must not overlap, as with the
// reference's kv_part_scratch, kvflash.cuh:56-69).  A call that finds the buffer large
// enough takes no lock.  When it has to grow, the new buffer is at least twice the old
// one and the old one is kept until the process ends (a call still in flight may be
// using it, and freeing it would mean draining the device under the lock): what the
// library ever holds per device stays below twice the largest request.
constexpr int MAX_DEVICES = 64;
std::mutex g_scratch_mu;
std::atomic<float*> g_scratch[MAX_DEVICES] = {};
std::atomic<size_t> g_scratch_cap[MAX_DEVICES] = {};

hipError_t scratch_floats(size_t n, float** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (dev < 0 || dev >= MAX_DEVICES) return hipErrorInvalidDevice;
  if (n <= g_scratch_cap[dev].load(std::memory_order_acquire)) {
    // (the pointer published with this capacity, or a larger buffer published since)
    *out = g_scratch[dev].load(std::memory_order_acquire);
    return hipSuccess;
  }
  std::lock_guard<std::mutex> lk(g_scratch_mu);
  const size_t have = g_scratch_cap[dev].load(std::memory_order_relaxed);
  if (n > have) {
    const size_t want = n > 2 * have ? n : 2 * have;
    float* nb = nullptr;
    e = hipMalloc((void**)&nb, want * sizeof(float));
    if (e != hipSuccess) return e;
    g_scratch[dev].store(nb, std::memory_order_release);
    g_scratch_cap[dev].store(want, std::memory_order_release);
  }
  *out = g_scratch[dev].load(std::memory_order_relaxed);
  return hipSuccess;
}

int check_kv_common(int H, int S, int D, int gs, int G, const char* who) {
  static thread_local char buf[96];
#define KV(cond, text)                                   \
  do {                                                   \
    if (!(cond)) {                                       \
      snprintf(buf, sizeof buf, "%s: %s", who, text);    \
      return invalid(buf);                               \
    }                                                    \
  } while (0)
  KV(H >= 1 && S >= 1 && D >= 1, "bad dims");
  KV(D <= 512, "D exceeds the 512-element bound");
  KV(gs >= 8 && gs % 8 == 0, "gs must be a multiple of 8");
  KV(G == (D + gs - 1) / gs, "G inconsistent with D, gs");
#undef KV
  return W4_OK;
}

// ---- the entry point that allocates nothing --------------------------------------
// Split-S partials of w4_attention_w4_flash_gqa_noalloc live in this file-scope
// device array instead of the grow-only buffer above.  Every GPU the library runs
// on holds its own copy until the process ends; its address on a device is looked
// up once, with that device current, and only that address is ever handed to
// kernels (the array's name is a host-side handle, not a device address).
constexpr size_t NOALLOC_SCRATCH_FLOATS = (size_t)W4_NOALLOC_SCRATCH_BYTES / sizeof(float);
__device__ __align__(256) float scratch[NOALLOC_SCRATCH_FLOATS];

constexpr int NOALLOC_MAX_DEVICES = MAX_DEVICES;
std::mutex g_noalloc_mu;
std::atomic<float*> g_noalloc_ptr[NOALLOC_MAX_DEVICES] = {};

// Device address of `scratch` on the current device (looked up on first use; later
// calls take no lock).
hipError_t noalloc_scratch(float** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (dev < 0 || dev >= NOALLOC_MAX_DEVICES) return hipErrorInvalidDevice;
  float* have = g_noalloc_ptr[dev].load(std::memory_order_acquire);
  if (!have) {
    std::lock_guard<std::mutex> lk(g_noalloc_mu);
    have = g_noalloc_ptr[dev].load(std::memory_order_relaxed);
    if (!have) {
      e = hipGetSymbolAddress((void**)&have, HIP_SYMBOL(scratch));
      if (e != hipSuccess) return e;
      if (!have) return hipErrorInvalidSymbol;
      g_noalloc_ptr[dev].store(have, std::memory_order_release);
    }
  }
  *out = have;
  return hipSuccess;
}

int run_flash(w4k::FlashArgs& a, w4_stream stream, const char* what) {
  float* part = nullptr;
  hipError_t e = scratch_floats(w4k::flash_scratch_floats(a), &part);
  if (e != hipSuccess) return runtime("flash scratch", e);
  return done(what, w4k::launch_flash(a, part, (hipStream_t)stream));
}

}  // namespace

extern "C" {

const char* w4_last_error(void) { return g_msg; }

int w4_dispatch_mma_min_m(void) { return DISPATCH_MMA_MIN_M; }
// Compute units of the current device, 256 (an MI355X) when there is none to ask: the
// threshold functions are plain arithmetic and callable without a GPU.
static int dispatch_cus() {
  static std::atomic<int> cached[MAX_DEVICES] = {};
  int dev = -1, n = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) return 256;
  if (const int have = cached[dev].load(std::memory_order_relaxed)) return have;
  if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n < 1)
    return 256;
  cached[dev].store(n, std::memory_order_relaxed);
  return n;
}

int w4_dispatch_mma_min_m_for_gs(int N, int K, int gs) {
  if (K % 32 != 0 && K % 8 == 0 && (long long)N * K >= (1LL << 25)) return 2;
  if (K > 4096 && K <= 6144 && K % 128 == 0) return 2;  // 5.8 us against 6.3 at N = 4096, M = 2
  if (K > 4096 && K % 32 == 0) return 3;
  // wide matrices at K <= 4096: from about 45 M weights the resident-activation kernel is
  // ahead at M = 3 and 4 (N = 11008 / 14336, K = 4096, gs = 128 or 32: 8.6 - 8.9 / 9.5 - 9.8 us
  // against 9.5 - 9.8 / 11.2 - 11.5); N = 8192 still belongs to the vector kernel (6.8 - 6.9
  // against 7.6).  Group sizes that are no multiple of 32 go to the matrix cores' general
  // kernel, which is slower there (N = 11008, gs = 48, M = 4: 11.8 us against 11.3 on the
  // vector units): they keep the plain threshold.
  // (measured on 256 compute units as N * K >= 44 M; what matters is that the grid holds
  // more than about 2.6 16-row tiles of 4096 k per compute unit, so it scales with them)
  if (K % 32 == 0 && (gs <= 0 || gs % 32 == 0) &&
      (long long)N * K >= 172000LL * dispatch_cus())
    return 3;
  return DISPATCH_MMA_MIN_M;
}
int w4_dispatch_mma_min_m_for(int N, int K) { return w4_dispatch_mma_min_m_for_gs(N, K, 0); }

int w4_dispatch_mma_min_m_for_mx(int N, int K) {
  // two activation rows at long K other than 8192 (which has the four-rows vector kernel):
  // the K-split vector kernel decodes every element once per activation row
  // (N = 4096, K = 11008 / 14336: 9.9 / 11.5 us against 8.3 / 9.8)
  if (K > 4096 && K % 32 == 0 && K != 8192) return 2;
  return w4_dispatch_mma_min_m_for(N, K);
}

// ---- W4 ----------------------------------------------------------------------

int w4_dequant(const w4_packed_view* p, w4_half* w, w4_stream stream) {
  if (int rc = check_packed(p, "dequant")) return rc;
  REQUIRE(w != nullptr, "dequant: null pointer");
  REQUIRE((long long)p->N * ((p->K + 7) / 8) < (1LL << 31), "dequant: N*words(K) exceeds 2^31");
  return done("dequant", w4k::launch_dequant(w4k::view_of(*p), w, (hipStream_t)stream));
}

int w4_gemm_fused(const w4_packed_view* p, const w4_half* x, w4_half* c, int M,
                  w4_stream stream, w4_half* w_out) {
  if (int rc = check_packed(p, "fused")) return rc;
  REQUIRE(x && c, "fused: null pointer");
  REQUIRE(M >= 1, "fused: bad M");
  REQUIRE(M <= FUSED_MAX_M && p->N <= INT_MAX - 32, "fused: launch grid out of range");
  return done("fused_kernel",
              w4k::launch_gemm_simt(w4k::view_of(*p), x, c, M, (hipStream_t)stream, w_out));
}

int w4_gemm_mma(const w4_packed_view* p, const w4_half* x, w4_half* c, int M,
                w4_stream stream, w4_half* w_out) {
  if (int rc = check_packed(p, "mma")) return rc;
  REQUIRE(x && c, "mma: null pointer");
  REQUIRE(M >= 1, "mma: bad M");
  REQUIRE(M <= MMA_MAX_M && p->N <= INT_MAX - 64, "mma: launch grid out of range");
  return done("mma_kernel",
              w4k::launch_gemm_mfma(w4k::view_of(*p), x, c, M, (hipStream_t)stream, w_out));
}

int w4_gemm(const w4_packed_view* p, const w4_half* x, w4_half* c, int M, w4_stream stream,
            w4_half* w_out) {
  const int min_m = p ? w4_dispatch_mma_min_m_for_gs(p->N, p->K, p->gs) : DISPATCH_MMA_MIN_M;
  return M < min_m ? w4_gemm_fused(p, x, c, M, stream, w_out)
                   : w4_gemm_mma(p, x, c, M, stream, w_out);
}

// ---- MXFP4 ---------------------------------------------------------------------

int w4_dequant_mx(const w4_packed_mx_view* p, w4_half* w, w4_stream stream) {
  if (int rc = check_mx(p)) return rc;
  REQUIRE(w != nullptr, "mx dequant: null output");
  REQUIRE((long long)p->N * ((p->K + 7) / 8) < (1LL << 31),
          "mx dequant: N*words(K) exceeds 2^31");
  return done("dequant_mx", w4k::launch_dequant(w4k::view_of(*p), w, (hipStream_t)stream));
}

int w4_gemm_fused_mx(const w4_packed_mx_view* p, const w4_half* x, w4_half* c, int M,
                     w4_stream stream, w4_half* w_out) {
  if (int rc = check_mx(p)) return rc;
  REQUIRE(x && c, "mx fused: null pointer");
  REQUIRE(M >= 1, "mx fused: bad M");
  REQUIRE(M <= FUSED_MAX_M && p->N <= INT_MAX - 32, "mx fused: launch grid out of range");
  return done("fused_kernel_mx",
              w4k::launch_gemm_simt(w4k::view_of(*p), x, c, M, (hipStream_t)stream, w_out));
}

int w4_gemm_mma_mx(const w4_packed_mx_view* p, const w4_half* x, w4_half* c, int M,
                   w4_stream stream, w4_half* w_out) {
  if (int rc = check_mx(p)) return rc;
  REQUIRE(x && c, "mx mma: null pointer");
  REQUIRE(M >= 1, "mx mma: bad M");
  REQUIRE(M <= MMA_MAX_M && p->N <= INT_MAX - 64, "mx mma: launch grid out of range");
  return done("mma_kernel_mx",
              w4k::launch_gemm_mfma(w4k::view_of(*p), x, c, M, (hipStream_t)stream, w_out));
}

int w4_gemm_mx(const w4_packed_mx_view* p, const w4_half* x, w4_half* c, int M,
               w4_stream stream, w4_half* w_out) {
  const int min_m = p ? w4_dispatch_mma_min_m_for_mx(p->N, p->K) : DISPATCH_MMA_MIN_M;
  return M < min_m ? w4_gemm_fused_mx(p, x, c, M, stream, w_out)
                   : w4_gemm_mma_mx(p, x, c, M, stream, w_out);
}

// ---- attention -------------------------------------------------------------------

static int check_kv_w4(const w4_kv_view* p, const char* who) {
  REQUIRE(p != nullptr, "kv flash: null view");
  if (int rc = check_kv_common(p->H, p->S, p->D, p->gs, p->G, who)) return rc;
  REQUIRE(p->q_k && p->s_k && p->q_v && p->s_v, "kv flash: null pointer");
  REQUIRE(p->symmetric || (p->z_k && p->z_v), "kv flash: asymmetric without zeros");
  REQUIRE(!p->symmetric || (!p->z_k && !p->z_v), "kv flash: symmetric carries no zeros");
  REQUIRE(p->S <= 65535 * 256, "kv flash: S exceeds the tile-grid bound");
  return W4_OK;
}

static void fill_w4(w4k::FlashArgs& a, const w4_kv_view* p, int group) {
  a = w4k::FlashArgs{};
  a.kind = 1;
  a.H = p->H; a.S = p->S; a.D = p->D; a.gs = p->gs; a.G = p->G;
  a.symmetric = p->symmetric;
  a.group = group;
  a.k = p->q_k; a.v = p->q_v; a.s_k = p->s_k; a.s_v = p->s_v;
  a.z_k = p->z_k; a.z_v = p->z_v;
  a.Hkv = p->H;
}

int w4_attention_w4_flash_gqa(const w4_kv_view* p, int group, const w4_half* q, w4_half* out,
                              w4_stream stream, w4_half* k_out, w4_half* v_out) {
  if (int rc = check_kv_w4(p, "kv flash")) return rc;
  REQUIRE(q && out, "kv flash w4: null pointer");
  REQUIRE(group >= 1 && group <= 64, "kv flash w4: bad query group");
  w4k::FlashArgs a;
  fill_w4(a, p, group);
  a.q = q; a.out = out; a.k_out = k_out; a.v_out = v_out;
  return run_flash(a, stream, "flash_w4");
}

int w4_attention_w4_flash_gqa_noalloc(const w4_kv_view* p, int group, const w4_half* q,
                                      w4_half* out, w4_stream stream, w4_half* k_out,
                                      w4_half* v_out) {
  if (int rc = check_kv_w4(p, "kv flash")) return rc;
  REQUIRE(q && out, "kv flash w4: null pointer");
  REQUIRE(group >= 1 && group <= 64, "kv flash w4: bad query group");
  w4k::FlashArgs a;
  fill_w4(a, p, group);
  a.q = q; a.out = out; a.k_out = k_out; a.v_out = v_out;
  // Same kernels and the same split plan as w4_attention_w4_flash_gqa: only where
  // the partials live differs, so the two give the same output bytes.  Phase 1
  // writes every partial phase 2 reads, so nothing needs clearing between calls.
  REQUIRE(w4k::flash_scratch_floats(a) <= NOALLOC_SCRATCH_FLOATS,
          "kv flash w4 noalloc: split-S partials exceed the built-in scratch "
          "(heads * group * splits * (D + 2) floats must fit W4_NOALLOC_SCRATCH_BYTES)");
  float* part = nullptr;
  hipError_t e = noalloc_scratch(&part);
  if (e != hipSuccess) return runtime("flash noalloc scratch", e);
  return done("flash_w4", w4k::launch_flash(a, part, (hipStream_t)stream));
}

int w4_attention_w4_flash(const w4_kv_view* p, const w4_half* q, w4_half* out,
                          w4_stream stream, w4_half* k_out, w4_half* v_out) {
  return w4_attention_w4_flash_gqa(p, 1, q, out, stream, k_out, v_out);
}

int w4_attention_fp16_flash_gqa(const w4_half* q, const w4_half* k16, const w4_half* v16,
                                w4_half* out, int H, int group, int S, int D,
                                w4_stream stream) {
  REQUIRE(H >= 1 && S >= 1 && D >= 1, "kv flash fp16: bad dims");
  REQUIRE(D <= 512, "kv flash fp16: D exceeds the 512-element bound");
  REQUIRE(S <= 65535 * 256, "kv flash fp16: S exceeds the tile-grid bound");
  REQUIRE(q && k16 && v16 && out, "kv flash fp16: null pointer");
  REQUIRE(group >= 1 && group <= 64, "kv flash fp16: bad query group");
  w4k::FlashArgs a{};
  a.kind = 0;
  a.H = H; a.S = S; a.D = D; a.gs = 8; a.G = 1; a.symmetric = 1; a.group = group;
  a.k = k16; a.v = v16; a.Hkv = H;
  a.q = q; a.out = out;
  return run_flash(a, stream, "flash_fp16");
}

int w4_attention_fp16_flash(const w4_half* q, const w4_half* k16, const w4_half* v16,
                            w4_half* out, int H, int S, int D, w4_stream stream) {
  return w4_attention_fp16_flash_gqa(q, k16, v16, out, H, 1, S, D, stream);
}

int w4_attention_f8_flash_gqa(const w4_kv_f8_view* p, int group, int scale_mode,
                              const w4_half* q, w4_half* out, w4_stream stream,
                              w4_half* k_out, w4_half* v_out) {
  REQUIRE(p != nullptr, "kv f8 flash: null view");
  if (int rc = check_kv_common(p->H, p->S, p->D, p->gs, p->G, "kv f8 flash")) return rc;
  REQUIRE(p->q_k && p->s_k && p->q_v && p->s_v, "kv f8 flash: null pointer");
  REQUIRE(p->S <= 65535 * 256, "kv f8 flash: S exceeds the tile-grid bound");
  REQUIRE(q && out, "kv f8 flash: null io pointer");
  REQUIRE(p->D % 4 == 0, "kv f8 flash: D must be a multiple of 4");
  REQUIRE((uintptr_t)p->q_k % 4 == 0 && (uintptr_t)p->q_v % 4 == 0,
          "kv f8 flash: cache bases 4-byte aligned");
  REQUIRE(group >= 1 && group <= 64, "kv f8 flash: bad query group");
  REQUIRE(scale_mode == 0 || scale_mode == 1, "kv f8 flash: bad scale mode");
  w4k::FlashArgs a{};
  a.kind = 2;
  a.H = p->H; a.S = p->S; a.D = p->D; a.gs = p->gs; a.G = p->G; a.symmetric = 1;
  a.group = group; a.scale_mode = scale_mode;
  a.k = p->q_k; a.v = p->q_v; a.s_k = p->s_k; a.s_v = p->s_v; a.Hkv = p->H;
  a.q = q; a.out = out; a.k_out = k_out; a.v_out = v_out;
  return run_flash(a, stream, "flash_f8");
}

int w4_attention_f8_flash(const w4_kv_f8_view* p, const w4_half* q, w4_half* out,
                          w4_stream stream, w4_half* k_out, w4_half* v_out) {
  return w4_attention_f8_flash_gqa(p, 1, 0, q, out, stream, k_out, v_out);
}

static int check_paged(const w4_kv_view* p, const int* bt, int page, int npages) {
  REQUIRE(p != nullptr, "kv paged flash: null view");
  if (int rc = check_kv_common(p->H, p->S, p->D, p->gs, p->G, "kv paged flash")) return rc;
  REQUIRE(p->q_k && p->s_k && p->q_v && p->s_v && bt, "kv paged flash: null pointer");
  REQUIRE(p->symmetric || (p->z_k && p->z_v), "kv paged flash: asymmetric without zeros");
  REQUIRE(!p->symmetric || (!p->z_k && !p->z_v), "kv paged flash: symmetric carries zeros");
  REQUIRE(page >= 1 && npages >= 1 && (long long)npages * page >= (long long)p->S,
          "kv paged flash: bad page geometry");
  REQUIRE((long long)npages * page < (1LL << 31), "kv paged flash: pool rows exceed 2^31");
  REQUIRE(p->S <= 65535 * 256, "kv paged flash: S exceeds tile-grid bound");
  return W4_OK;
}

int w4_attention_w4_flash_paged(const w4_kv_view* p, const int* bt, int page, int npages,
                                const w4_half* q, w4_half* out, w4_stream stream,
                                w4_half* k_out, w4_half* v_out) {
  if (int rc = check_paged(p, bt, page, npages)) return rc;
  REQUIRE(q && out, "kv paged flash: null io");
  w4k::FlashArgs a;
  fill_w4(a, p, 1);
  a.bt = bt; a.bt_stride = 0; a.page = page; a.pool_rows = npages * page;
  a.Hkv = p->H;  // one table for every head: sequence index is always 0
  a.q = q; a.out = out; a.k_out = k_out; a.v_out = v_out;
  return run_flash(a, stream, "flash_w4_paged");
}

int w4_attention_w4_flash_paged_batched(const w4_kv_view* p, const int* bt, int nseq,
                                        int bt_stride, int page, int npages, int group,
                                        const w4_half* q, w4_half* out, w4_stream stream) {
  if (int rc = check_paged(p, bt, page, npages)) return rc;
  REQUIRE(q && out, "kv paged flash: null io");
  REQUIRE(nseq >= 1 && group >= 1 && group <= 64, "kv paged flash: bad batch");
  REQUIRE(bt_stride >= (p->S + page - 1) / page, "kv paged flash: table stride too short");
  REQUIRE((long long)nseq * p->H < (1LL << 31), "kv paged flash: too many slabs");
  w4k::FlashArgs a;
  fill_w4(a, p, group);
  a.H = nseq * p->H;
  a.Hkv = p->H;
  a.bt = bt; a.bt_stride = bt_stride; a.page = page; a.pool_rows = npages * page;
  a.q = q; a.out = out;
  return run_flash(a, stream, "flash_w4_paged");
}

int w4_dequant_f8(const uint8_t* q, const w4_half* s, w4_half* w, int S, int D, int gs,
                  w4_stream stream) {
  REQUIRE(S >= 1 && D >= 1, "f8 dequant: bad dims");
  REQUIRE(gs >= 8 && gs % 8 == 0, "f8 dequant: gs must be a multiple of 8");
  REQUIRE(q && s && w, "f8 dequant: null pointer");
  REQUIRE((long long)S * ((D + 3) / 4) < (1LL << 31), "f8 dequant: S*words4(D) exceeds 2^31");
  REQUIRE(D % 4 == 0, "f8 dequant: D must be a multiple of 4");
  REQUIRE((uintptr_t)q % 4 == 0, "f8 dequant: q must be 4-byte aligned");
  return done("dequant_f8", w4k::launch_dequant_f8(q, s, w, S, D, gs, (hipStream_t)stream));
}

// ---- device-side quantizers -------------------------------------------------------
// Contracts of the host quantizers (pack.hpp:64-72, mx.hpp:71-76,
// kvcache.hpp:60-68, kvfp8.hpp:70-79); what they find in the data (non-finite
// input, scale out of range) lands in *status instead of a throw.

static int start_status(int* status, w4_stream stream, const char* what) {
  return done(what, w4k::launch_fill_words((uint32_t*)status, 1, 0u, (hipStream_t)stream));
}

int w4_quantize(const w4_packed_view* out, const double* w, int* status, w4_stream stream) {
  if (int rc = check_packed(out, "quantize")) return rc;
  REQUIRE(w && status, "quantize: null pointer");
  if (int rc = start_status(status, stream, "quantize")) return rc;
  const w4k::QuantSide side{w, (uint32_t*)out->q, nullptr, (w4_half*)out->scales,
                            (uint32_t*)out->zeros};
  return done("quantize", w4k::launch_quantize_rows(out->symmetric ? 0 : 1, &side, 1, 0, out->N,
                                                    out->K, out->gs, status, (hipStream_t)stream));
}

int w4_quantize_mx(const w4_packed_mx_view* out, const double* w, int* status,
                   w4_stream stream) {
  REQUIRE(out != nullptr, "quantize_mx: null view");
  REQUIRE(out->N >= 1 && out->K >= 1, "quantize_mx: bad dims");
  REQUIRE(out->B == (out->K + 31) / 32, "quantize_mx: B inconsistent with K");
  REQUIRE(out->q && out->scales && w && status, "quantize_mx: null pointer");
  if (int rc = start_status(status, stream, "quantize_mx")) return rc;
  return done("quantize_mx",
              w4k::launch_quantize_mx(w, 0, out->N, out->K, (uint32_t*)out->q,
                                      (uint8_t*)out->scales, status, (hipStream_t)stream));
}

int w4_quantize_mx_f16(const w4_packed_mx_view* out, const w4_half* x, int* status,
                       w4_stream stream) {
  REQUIRE(out != nullptr, "quantize_mx: null view");
  REQUIRE(out->N >= 1 && out->K >= 1, "quantize_mx: bad dims");
  REQUIRE(out->B == (out->K + 31) / 32, "quantize_mx: B inconsistent with K");
  REQUIRE(out->q && out->scales && x && status, "quantize_mx: null pointer");
  if (int rc = start_status(status, stream, "quantize_mx")) return rc;
  return done("quantize_mx",
              w4k::launch_quantize_mx(x, 1, out->N, out->K, (uint32_t*)out->q,
                                      (uint8_t*)out->scales, status, (hipStream_t)stream));
}

// ---- W4A4 on the scaled matrix cores ---------------------------------------------

int w4_gemm_mx_w4a4(const w4_packed_mx_view* w, const w4_packed_mx_view* x, w4_half* c,
                    w4_stream stream) {
  if (int rc = check_mx(w)) return rc;
  if (int rc = check_mx(x)) return rc;
  REQUIRE(w->K == x->K, "mx w4a4: operands disagree on K");
  REQUIRE(c != nullptr, "mx w4a4: null pointer");
  REQUIRE(x->N <= 65535LL * 64, "mx w4a4: launch grid out of range");
  return done("gemm_mx_w4a4", w4k::launch_gemm_mx_w4a4(*w, *x, c, (hipStream_t)stream));
}

static int check_mx8(const w4_act_mx8_view* p) {
  REQUIRE(p != nullptr, "mx8: null view");
  REQUIRE(p->M >= 1 && p->K >= 1, "mx8: bad dims");
  REQUIRE(p->B == (p->K + 31) / 32, "mx8: B inconsistent with K");
  REQUIRE(p->q && p->scales, "mx8: null pointer");
  return W4_OK;
}

int w4_quantize_mx8_f16(const w4_act_mx8_view* out, const w4_half* x, int* status,
                        w4_stream stream) {
  if (int rc = check_mx8(out)) return rc;
  REQUIRE(x && status, "quantize_mx8: null pointer");
  if (int rc = start_status(status, stream, "quantize_mx8")) return rc;
  return done("quantize_mx8",
              w4k::launch_quantize_mx8(x, 1, out->M, out->K, (uint8_t*)out->q,
                                       (uint8_t*)out->scales, status, (hipStream_t)stream));
}

int w4_gemm_mx_w4a8(const w4_packed_mx_view* w, const w4_act_mx8_view* x, w4_half* c,
                    w4_stream stream) {
  if (int rc = check_mx(w)) return rc;
  if (int rc = check_mx8(x)) return rc;
  REQUIRE(w->K == x->K, "mx w4a8: operands disagree on K");
  REQUIRE(w->K % 32 == 0, "mx w4a8: K must be a multiple of 32");
  REQUIRE(((uintptr_t)x->q & 15) == 0, "mx w4a8: x must be 16-byte aligned");
  REQUIRE(c != nullptr, "mx w4a8: null pointer");
  REQUIRE(x->M <= 65535LL * 64, "mx w4a8: launch grid out of range");
  return done("gemm_mx_w4a8", w4k::launch_gemm_mx_w4a8(*w, *x, c, (hipStream_t)stream));
}

int w4_quantize_cache(const w4_kv_view* out, const void* k, const void* v, int src_f16,
                      int* status, w4_stream stream) {
  REQUIRE(out != nullptr, "quantize_cache: null view");
  REQUIRE(out->H >= 1 && out->S >= 1 && out->D >= 1, "quantize_cache: bad dims");
  REQUIRE(out->gs >= 8 && out->gs % 8 == 0, "quantize_cache: gs must be a multiple of 8");
  REQUIRE(out->G == (out->D + out->gs - 1) / out->gs, "quantize_cache: G inconsistent with D, gs");
  REQUIRE(out->q_k && out->s_k && out->q_v && out->s_v && k && v && status,
          "quantize_cache: null pointer");
  REQUIRE(out->symmetric || (out->z_k && out->z_v), "quantize_cache: asymmetric without zeros");
  REQUIRE(!out->symmetric || (!out->z_k && !out->z_v),
          "quantize_cache: symmetric carries no zeros");
  if (int rc = start_status(status, stream, "quantize_cache")) return rc;
  const w4k::QuantSide sides[2] = {
      {k, (uint32_t*)out->q_k, nullptr, (w4_half*)out->s_k, (uint32_t*)out->z_k},
      {v, (uint32_t*)out->q_v, nullptr, (w4_half*)out->s_v, (uint32_t*)out->z_v}};
  return done("quantize_cache",
              w4k::launch_quantize_rows(out->symmetric ? 0 : 1, sides, 2, src_f16,
                                        (long long)out->H * out->S, out->D, out->gs, status,
                                        (hipStream_t)stream));
}

int w4_quantize_cache_f8(const w4_kv_f8_view* out, const void* k, const void* v, int src_f16,
                         int* status, w4_stream stream) {
  REQUIRE(out != nullptr, "quantize_cache_f8: null view");
  REQUIRE(out->H >= 1 && out->S >= 1 && out->D >= 1, "quantize_cache_f8: bad dims");
  REQUIRE(out->gs >= 8 && out->gs % 8 == 0, "quantize_cache_f8: gs must be a multiple of 8");
  REQUIRE(out->G == (out->D + out->gs - 1) / out->gs,
          "quantize_cache_f8: G inconsistent with D, gs");
  REQUIRE(out->q_k && out->s_k && out->q_v && out->s_v && k && v && status,
          "quantize_cache_f8: null pointer");
  if (int rc = start_status(status, stream, "quantize_cache_f8")) return rc;
  const w4k::QuantSide sides[2] = {{k, nullptr, (uint8_t*)out->q_k, (w4_half*)out->s_k, nullptr},
                                   {v, nullptr, (uint8_t*)out->q_v, (w4_half*)out->s_v, nullptr}};
  return done("quantize_cache_f8",
              w4k::launch_quantize_rows(2, sides, 2, src_f16, (long long)out->H * out->S, out->D,
                                        out->gs, status, (hipStream_t)stream));
}

}  // extern "C"

// ---- two-pass baseline -------------------------------------------------------------
extern "C" int w4_gemm_fp16_impl(const w4_half*, const w4_half*, w4_half*, int, int, int,
                                 w4_stream);
extern "C" const char* w4_blas_last_error(void);

extern "C" int w4_gemm_fp16(const w4_half* w, const w4_half* x, w4_half* c, int M, int N,
                            int K, w4_stream stream) {
  REQUIRE(M >= 1 && N >= 1 && K >= 1, "gemm_fp16: bad dims");
  REQUIRE(w && x && c, "gemm_fp16: null pointer");
  const int rc = w4_gemm_fp16_impl(w, x, c, M, N, K, stream);
  if (rc != W4_OK) snprintf(g_msg, sizeof g_msg, "%s", w4_blas_last_error());
  return rc;
}
